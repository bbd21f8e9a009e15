"""Resolve the references a claim names (a state hook, a proof gate) to code that exists in the tree.

Reference: isoexec/core/claim_refs.py:19-76. Paths are containment-checked so a ``../`` reference
cannot reach outside the package, and symbols are found by parsing rather than by text search.
Gates are the parity tests: the package's own ``ops/*/tests`` and the repository's ``tests`` folder.
"""

from __future__ import annotations

import ast
import pathlib

PACKAGE_DIR = pathlib.Path(__file__).resolve().parents[1]
_GATE_GLOBS = ((PACKAGE_DIR, "ops/*/tests/*.py"), (PACKAGE_DIR.parents[1], "tests/*.py"))
_gate_text: dict | None = None


def _inside_package(path: str):
    try:
        full = (PACKAGE_DIR / path).resolve()
        full.relative_to(PACKAGE_DIR)
        return full
    except (ValueError, OSError):
        return None


def _top_level_names(source: str) -> set:
    try:
        body = ast.parse(source).body
    except SyntaxError:
        return set()
    return {n.name for n in body if isinstance(n, (ast.FunctionDef, ast.AsyncFunctionDef, ast.ClassDef))}


def hook_ref_problem(ref: str):
    """Why ``path::symbol`` names no code in this package, or None when it does."""
    path, _, symbol = ref.partition("::")
    target = _inside_package(path)
    if target is None:
        return f"ref path {path!r} escapes the package, so it names no code this tree ships"
    if not target.is_file():
        return f"ref file {path!r} missing"
    if symbol not in _top_level_names(target.read_text(errors="replace")):
        return f"hook {symbol!r} not defined in {path}"
    return None


def _gates() -> dict:
    global _gate_text
    if _gate_text is None:
        _gate_text = {}
        for root, pattern in _GATE_GLOBS:
            for p in sorted(root.glob(pattern)):
                _gate_text[str(p.relative_to(root))] = p.read_text(errors="replace")
    return _gate_text


def proof_ref_problem(ref: str):
    """Why a proof pointer resolves to no gate, or None when it does. The pointer is a path inside
    the package, or ``"<gate name>: <what it shows>"`` where the name appears in a gate's path or text."""
    words = ref.strip().split(":")[0].split()
    if not words:
        return "empty proof ref"
    name = words[0]
    target = _inside_package(name)
    if target is not None and target.is_file():
        return None
    if any(name in path or name in text for path, text in _gates().items()):
        return None
    return f"proof ref {ref!r} resolves to no gate: {name!r} names no file and appears in no test source"

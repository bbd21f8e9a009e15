"""Does a reference written into a claim point at something that exists?

Two kinds of reference appear in a contract: ``file.py::symbol`` for the hook that implements a state claim, and a
proof pointer for an invariance or equivalence claim, which names a gate (a parity test) either by file or by a word
that occurs in a gate. Files are looked up inside this package only (a path that climbs out of it is refused), and a
symbol counts only if the file defines it at module level -- a mention in a comment does not. Gates are the
package's ``ops/*/tests`` and the repository's ``tests`` folder. (Reference: isoexec/core/claim_refs.py:19-76.)
"""

from __future__ import annotations

import ast
from pathlib import Path
from typing import Dict, Optional

PACKAGE_DIR = Path(__file__).resolve().parent.parent
_REPO_DIR = PACKAGE_DIR.parent.parent


class _GateIndex:
    """Path and text of every gate file, read on first use."""

    where = ((PACKAGE_DIR, "ops/*/tests/*.py"), (_REPO_DIR, "tests/*.py"))

    def __init__(self):
        self._files: Optional[Dict[str, str]] = None

    def mentions(self, word: str) -> bool:
        if self._files is None:
            self._files = {}
            for base, pattern in self.where:
                for f in sorted(base.glob(pattern)):
                    self._files[f.relative_to(base).as_posix()] = f.read_text(errors="replace")
        return any(word in name or word in text for name, text in self._files.items())


_gates = _GateIndex()


def _package_file(relative: str) -> Optional[Path]:
    """``relative`` as a path under the package, or None if it leaves the package or cannot be resolved."""
    try:
        candidate = (PACKAGE_DIR / relative).resolve()
    except OSError:
        return None
    return candidate if PACKAGE_DIR in candidate.parents or candidate == PACKAGE_DIR else None


def _module_level_definitions(path: Path) -> set:
    try:
        module = ast.parse(path.read_text(errors="replace"))
    except SyntaxError:
        return set()
    kinds = (ast.FunctionDef, ast.AsyncFunctionDef, ast.ClassDef)
    return {node.name for node in module.body if isinstance(node, kinds)}


def hook_ref_problem(ref: str) -> Optional[str]:
    """None if ``path::symbol`` names a definition in this package, else what is wrong with it."""
    relative, _sep, symbol = ref.partition("::")
    path = _package_file(relative)
    if path is None:
        return f"ref path {relative!r} escapes the package, so it names no code this tree ships"
    if not path.is_file():
        return f"ref file {relative!r} missing"
    if symbol in _module_level_definitions(path):
        return None
    return f"hook {symbol!r} not defined in {relative}"


def proof_ref_problem(ref: str) -> Optional[str]:
    """None if the pointer resolves to a gate, else why not. A pointer is a file path inside the package, or
    ``"<gate word>: <what the gate shows>"``; only the first word before the colon is looked up."""
    head = ref.strip().partition(":")[0].split()
    if not head:
        return "empty proof ref"
    word = head[0]
    path = _package_file(word)
    if (path is not None and path.is_file()) or _gates.mentions(word):
        return None
    return f"proof ref {ref!r} resolves to no gate: {word!r} names no file and appears in no test source"

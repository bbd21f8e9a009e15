"""Registry + ``{(op, site): selection}`` -> a frozen, validated ExecutionContract.

Reference: isoexec/core/contract_build.py:37-435. The build runs in four passes:

1. admit    every key names a registered op, a site that op declares, a registered impl, and an impl
            whose ``supported_archs`` contains the arch being built for;
2. pins     every pinned constant is a key the impl's rounding schedule declares, with a value the
            schedule allows (a pin nobody checks would hash and match while constraining nothing);
3. project  per op, sites with an identical selection merge into one entry whose region is the op plus
            whatever its impl subsumes; an op that resolves to several impls gets the discharge that
            licenses the whole group; float pins travel as fp64 bit patterns;
4. freeze   the three identities are computed and the structural rules checked.
"""

from __future__ import annotations

import dataclasses
import json
import struct
from collections.abc import Mapping
from typing import Dict, Optional

from .. import contract as K
from . import claim_refs
from .arch import ARCH, HardwareTarget, is_accelerator_arch
from .registry import Registry, RegistryError

FUNCTION = "function"      # hashed into numerical_policy
DEPLOYMENT = "deployment"  # proven bitwise-neutral; hashed into the deployment identity only

# The four execution cases a site name stands for (reference: contract_build.py:41-53).
CASES = (
    K.ExecutionCase(
        "engine_decode", "engine", "no_grad", "continued", "shape_static",
        ("cudagraph_capturable", "host_free", "address_stable"),
    ),
    K.ExecutionCase("engine_prefill", "engine", "no_grad", "resumable", "variable"),
    K.ExecutionCase("trainer_fwd", "trainer", "grad", "checkpoint_recompute", "variable", ("includes_grad_recompute",)),
    K.ExecutionCase("trainer_score", "trainer", "no_grad", "fresh", "variable"),
)


class ContractBuildError(ValueError):
    pass


class PinValidationError(ContractBuildError):
    """Pinned constants disagree with the selected impl's declared rounding schedule."""


@dataclasses.dataclass(frozen=True)
class _Choice:
    impl_id: str
    version: int
    pinned_constants: dict
    classification: str
    neutrality_proof: Optional[str]

    def bucket(self) -> str:
        # Sites merge when this text is equal.
        return json.dumps(
            [self.impl_id, self.version, self.pinned_constants, self.classification, self.neutrality_proof],
            sort_keys=True,
            default=str,
        )


def _choice(op: str, site: str, raw) -> _Choice:
    """Normalise a selection given as a record (attribute access) or as a plain mapping."""
    if isinstance(raw, Mapping):
        read = lambda name, default=None: raw.get(name, default)  # noqa: E731
        impl_id = raw["impl_id"]
    else:
        read = lambda name, default=None: getattr(raw, name, default)  # noqa: E731
        impl_id = raw.impl_id
    c = _Choice(
        impl_id=impl_id,
        version=read("version", 1),
        pinned_constants=dict(read("pinned_constants") or {}),
        classification=read("classification", FUNCTION),
        neutrality_proof=read("neutrality_proof"),
    )
    where = f"({op}, {site})"
    if c.classification not in (FUNCTION, DEPLOYMENT):
        raise ContractBuildError(
            f"{where}: unknown classification {c.classification!r}; must be one of ['{DEPLOYMENT}', '{FUNCTION}']"
        )
    if c.classification == DEPLOYMENT and not c.neutrality_proof:
        raise ContractBuildError(
            f"{where}: deployment classification requires a recorded neutrality_proof (a run id or gate "
            "result). A neutrality proof licenses exactly the entry it was measured on."
        )
    if c.classification == FUNCTION and c.neutrality_proof:
        raise ContractBuildError(
            f"{where}: a function-half entry must not carry a neutrality_proof; classify it deployment "
            "if it is proven neutral, otherwise leave it function without one."
        )
    return c


def validate_pins(registry: Registry, selections: Dict, model: Optional[str] = None) -> None:
    """Refuse pins the selected impl never declared or contradicts; every offender is named at once."""
    bad = []
    for (op, site), raw in sorted(selections.items()):
        c = raw if isinstance(raw, _Choice) else _choice(op, site, raw)
        if not registry.has_op(op):
            if c.pinned_constants:
                bad.append(f"({op}, {site}): op is not registered, so its pins cannot be checked")
            continue
        impl = registry.get_op(op).impls.get(c.impl_id)
        if impl is None:
            if c.pinned_constants:
                bad.append(f"({op}, {site}): impl {c.impl_id!r} is not registered on the op")
            continue
        for key in sorted(c.pinned_constants, key=str):
            why = impl.rounding.check_pin(key, c.pinned_constants[key])
            if why:
                bad.append(
                    f"({op}, {site}) impl {c.impl_id}@v{impl.version}: pin {key}={c.pinned_constants[key]!r} -- {why}"
                )
    if bad:
        subject = f"model {model!r}" if model else "selections"
        raise PinValidationError(
            f"{subject}: pinned constants disagree with the selected impls' declared rounding schedules:\n  "
            + "\n  ".join(bad)
            + "\n\nA pinned constant is a claim about the FUNCTION the composition names. Unchecked, it "
            "hashes identically on both runtimes, so agreement stays green while the composition names "
            "the wrong function. Fix the profile or the impl's schedule; do not drop the pin and do not "
            "weaken the schedule to make this pass."
        )


def _wire_constant(op: str, key: str, value):
    if value is None or isinstance(value, (bool, int, str)):
        return value
    if isinstance(value, float):
        (bits,) = struct.unpack("<Q", struct.pack("<d", value))
        return K.BitPattern("0x%016x" % bits, "fp64")
    raise ContractBuildError(f"({op}) pin {key!r}: non-scalar pin values are not projectable")


class _Discharger:
    """Finds the claim that licenses an op resolving to more than one impl across its sites."""

    def __init__(self, registry: Registry, op: str, choices: dict):
        self.registry, self.op, self.choices = registry, op, choices
        self.impl_ids = sorted({c.impl_id for c in choices.values()})

    def _spec(self, impl_id):
        return self.registry.get_op(self.op).impls.get(impl_id) if self.registry.has_op(self.op) else None

    def _bitwise_claims(self) -> dict:
        claims = {}
        for impl_id in self.impl_ids:
            spec = self._spec(impl_id)
            twin = spec.capabilities.get("bitwise_equal_to") if spec else None
            if twin is None:
                continue
            if twin == impl_id:
                raise ContractBuildError(
                    f"op {self.op!r}: impl {impl_id!r} declares bitwise_equal_to ITSELF. A self-claim "
                    f"discharges nothing; name the sibling it was compared against."
                )
            if self._spec(twin) is None:
                raise ContractBuildError(
                    f"op {self.op!r}: impl {impl_id!r} declares bitwise_equal_to={twin!r}, which is not a "
                    f"registered impl of this op (registered: {sorted(self.registry.get_op(self.op).impls)})."
                )
            if twin not in self.impl_ids:
                raise ContractBuildError(
                    f"op {self.op!r}: impl {impl_id!r} declares bitwise_equal_to={twin!r}, but this "
                    f"composition selects {self.impl_ids}; the claim does not reach the impls in the group."
                )
            claims[impl_id] = twin
        return claims

    def resolve(self):
        if len(self.impl_ids) <= 1:
            return None
        claims = self._bitwise_claims()
        if claims:
            # Union the claimed pairs; the group is licensed only if they connect every selected impl.
            root = {i: i for i in self.impl_ids}

            def find(i):
                while root[i] != i:
                    i = root[i]
                return i

            for a, b in claims.items():
                root[find(a)] = find(b)
            anchor = find(self.impl_ids[0])
            reached = sorted(i for i in self.impl_ids if find(i) == anchor)
            if len(reached) != len(self.impl_ids):
                raise ContractBuildError(
                    f"op {self.op!r} resolves to {self.impl_ids} across sites, but the declared "
                    f"bitwise_equal_to claims {claims} link only {reached}: "
                    f"{sorted(set(self.impl_ids) - set(reached))} carry no discharge."
                )
            return K.EquivalenceProof("bitwise_equal_to", claims[min(claims)])
        for impl_id in self.impl_ids:
            spec = self._spec(impl_id)
            proof = spec.capabilities.get("equivalence_proof") if spec else None
            if proof:
                problem = claim_refs.proof_ref_problem(proof)
                if problem:
                    raise ContractBuildError(
                        f"op {self.op!r}: impl {impl_id!r} declares an equivalence_proof but {problem}. "
                        f"Name the gate that measured the property."
                    )
                return K.EquivalenceProof("equivalence_proof", proof)
        neutral = {c.neutrality_proof for c in self.choices.values() if c.classification == DEPLOYMENT}
        if len(neutral) == 1:
            return K.EquivalenceProof("neutrality_proof", neutral.pop())
        raise ContractBuildError(
            f"op {self.op!r} resolves to {self.impl_ids} across sites but no selected impl declares "
            f"bitwise_equal_to / equivalence_proof and no single neutrality proof licenses the group"
        )


def derive_topology_claims(topology) -> tuple:
    """Profile topology facts -> claims, in axis order so declaration order never moves a hash."""
    return tuple(
        K.TopologyClaim(t.axis, t.kind, t.degree, t.collective_plan, tuple(t.domain), t.proof)
        for t in sorted(topology or (), key=lambda t: t.axis)
    )


def derive_state_claims(states) -> tuple:
    return tuple(
        K.StateClaim(s.state_id, tuple(s.invalidated_by), bool(s.replay_safe), s.ref)
        for s in sorted(states or (), key=lambda s: s.state_id)
    )


def derive_tolerance_claims(tolerances) -> tuple:
    return tuple(
        K.ToleranceClaim(tuple(t.case_pair), tuple(t.bounds), tuple(t.attributed_to))
        for t in sorted(tolerances or (), key=lambda t: t.case_pair)
    )


def _admit(registry: Registry, selections: Dict, arch: str) -> Dict:
    target = HardwareTarget(arch)
    admitted = {}
    for (op, site), raw in selections.items():
        if not registry.has_op(op):
            raise ContractBuildError(f"selection names unknown op {op!r} (not in registry)")
        spec = registry.get_op(op)
        if site not in spec.sites:
            raise ContractBuildError(
                f"selection names site {site!r} for op {op!r}, but that op declares only "
                f"{sorted(spec.sites)} (absence means 'no such site')"
            )
        c = _choice(op, site, raw)
        impl = spec.impls.get(c.impl_id)
        if impl is None:
            raise ContractBuildError(
                f"selection for ({op!r}, {site!r}) names impl {c.impl_id!r} not registered on the op "
                f"(known: {sorted(spec.impls)})"
            )
        # Evidence is arch-scoped. Skipped only under the sentinel, which names no accelerator.
        if is_accelerator_arch(arch) and not target.supports(impl.supported_archs):
            raise ContractBuildError(
                f"selection for ({op!r}, {site!r}) names impl {c.impl_id!r}, which declares "
                f"supported_archs {sorted(impl.supported_archs)}, but this contract is being built for "
                f"arch {arch!r}. The identity would be keyed to an arch on which nothing was proven: "
                f"run the impl's parity battery on {arch!r} and declare it, or select an impl that supports it."
            )
        admitted[(op, site)] = c
    return admitted


def _project(registry: Registry, admitted: Dict, arch: str) -> list:
    per_op: Dict[str, Dict[str, _Choice]] = {}
    for (op, site), c in admitted.items():
        per_op.setdefault(op, {})[site] = c
    entries = []
    for op in sorted(per_op):
        by_site = per_op[op]
        group_proof = _Discharger(registry, op, by_site).resolve()
        merged: Dict[str, list] = {}
        for site, c in by_site.items():
            merged.setdefault(c.bucket(), []).append(site)
        for text in sorted(merged):
            sites = tuple(sorted(merged[text]))
            c = by_site[sites[0]]
            impl = registry.get_op(op).impls[c.impl_id]
            neutral = c.classification == DEPLOYMENT
            entries.append(
                K.CompositionEntry(
                    region=tuple(sorted((op, *impl.subsumes))),
                    cases=sites,
                    impl=K.ImplRef(c.impl_id, c.version, arch),
                    route=impl.route,
                    constants={k: _wire_constant(op, k, v) for k, v in c.pinned_constants.items()},
                    discharge=K.EquivalenceProof("neutrality_proof", c.neutrality_proof) if neutral else group_proof,
                    half=DEPLOYMENT if neutral else FUNCTION,
                )
            )
    entries.sort(key=lambda e: (e.region, e.cases, e.impl.id))
    return entries


_validate_pins = validate_pins


def build_execution_contract(
    registry: Registry,
    selections: Dict,
    arch: str = ARCH,
    model: Optional[str] = None,
    profile=None,
    topology=(),
    states=(),
    tolerances=(),
    validate_pins: bool = True,
    allow_non_accelerator_arch: bool = False,
) -> K.ExecutionContract:
    """The single build path. ``validate_pins=False`` exists for tests of the projection alone."""
    if not allow_non_accelerator_arch and not is_accelerator_arch(arch):
        raise ContractBuildError(
            f"refusing to build a contract whose arch is {arch!r}: that is the non-accelerator sentinel, "
            f"not a real accelerator key. Folding it into the identity would key every recorded signature "
            f"away from the real accelerator's table while hash cross-checks still pass. Build where the "
            f"accelerator is visible or pass an explicit arch; CPU-only tests that intend a sentinel "
            f"contract pass allow_non_accelerator_arch=True."
        )
    if not selections:
        raise ContractBuildError(
            "refusing to build a contract from an empty selection map: it would name no execution, and two "
            "processes that both failed to derive a composition would agree perfectly."
        )
    try:
        registry.assert_subsumption_closed()
    except RegistryError as exc:
        raise ContractBuildError(f"refusing to build against a registry that is not subsumption-closed: {exc}") from exc

    admitted = _admit(registry, selections, arch)
    if validate_pins:
        _validate_pins(registry, admitted, model=model)
    composition = tuple(_project(registry, admitted, arch))

    live_cases = {site for _, site in admitted}
    claims = K.Claims(
        topology=derive_topology_claims(topology),
        state=derive_state_claims(states),
        tolerances=derive_tolerance_claims(tolerances),
    )
    for t in claims.topology:
        problem = None if t.proof is None else claim_refs.proof_ref_problem(t.proof)
        if problem:
            raise ContractBuildError(f"topology claim {t.axis!r}: {problem}.")
    draft = K.ExecutionContract(
        schema_version="2",
        model=K.ModelRef(model or "", tuple(getattr(profile, "architectures", ()) or ()), f"models/{model or 'unknown'}"),
        identities=K.Identities("", "", ""),
        cases=tuple(c for c in CASES if c.id in live_cases),
        composition=composition,
        claims=claims,
    )
    frozen = K.freeze(draft)
    owned = {c.id: frozenset(op for e in composition if c.id in e.cases for op in e.region) for c in frozen.cases}
    K.validate_or_raise(frozen, required_ops=owned)
    return frozen

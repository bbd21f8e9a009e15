"""Registry entries for the RMS norms (reference: isoexec/ops/norms/_register.py)."""

from ...core.registry import ImplSpec, OpSpec, RoundingSchedule

SITES = ["trainer_fwd", "trainer_score", "engine_prefill", "engine_decode"]
GFX950 = frozenset({"gfx950"})

_SUMSQ = "8 per-lane column sums of rounded squares over chunks left to right, tree over the 8, then adjacent-pairwise lane tree"


def register(reg) -> None:
    reg.register_op(
        OpSpec(name="norms.rms", sites=list(SITES)).add_impl(
            ImplSpec(
                impl_id="hip_fused",
                version=1,
                supported_archs=GFX950,
                rounding=RoundingSchedule(
                    machine_assertable={
                        "compute_dtype": "fp32",
                        "sum_of_squares": _SUMSQ,
                        "fma": False,
                        "rsqrt": "1/sqrtf (IEEE divide of IEEE sqrt)",
                        "gamma": "x * rstd * (1 + w), each product rounded",
                        "residual_add": "rounded to the io dtype before the norm",
                    },
                    documentary=(
                        "Zero-centred RMS norm, optionally fused with the residual add. One wave-slice "
                        "per row; the reduction tree depends on the row width alone."
                    ),
                ),
                capabilities={"zero_centered": True, "fused_residual_add": True},
                hazards=["non_contiguous", "subnormals"],
            )
        )
    )
    reg.register_op(
        OpSpec(name="norms.gated_out", sites=list(SITES)).add_impl(
            ImplSpec(
                impl_id="hip_fused",
                version=1,
                supported_archs=GFX950,
                rounding=RoundingSchedule(
                    machine_assertable={
                        "compute_dtype": "fp32",
                        "sum_of_squares": _SUMSQ,
                        "fma": False,
                        "gate": "silu(z) = z / (1 + exp(-z)), multiplied after the norm",
                    },
                    documentary="RMS norm of the GatedDeltaNet output times gamma, then times silu(gate).",
                ),
                hazards=["non_contiguous"],
            )
        )
    )

"""Registry entry for rotary embedding (reference: isoexec/ops/rope/_register.py)."""

from ...core.registry import ImplSpec, OpSpec, RoundingSchedule

SITES = ["trainer_fwd", "trainer_score", "engine_prefill", "engine_decode"]


def register(reg) -> None:
    reg.register_op(
        OpSpec(name="rope.rope", sites=list(SITES)).add_impl(
            ImplSpec(
                impl_id="hip_rope",
                version=1,
                supported_archs=frozenset({"gfx950"}),
                rounding=RoundingSchedule(
                    machine_assertable={
                        "cos_sin_table": "float64 on the host, rounded to fp32 then bf16",
                        "mul_add_opmath": "bf16_three_rounds",
                        "rotate_half_negation": "mul_neg_one",
                        "fma": False,
                    },
                    documentary=(
                        "Rotate-half over the first R lanes: lane d takes lane d+R/2 negated below R/2 and "
                        "lane d-R/2 above; bf16(bf16(x*cos) + bf16(rot*sin)). Elementwise, so no order to pin."
                    ),
                ),
                hazards=["signed_zero", "non_contiguous"],
            )
        )
    )

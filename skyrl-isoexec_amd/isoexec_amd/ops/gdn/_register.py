"""Registry entries for the GatedDeltaNet family (reference: isoexec/ops/gdn/_register.py)."""

from ...core.registry import ImplSpec, OneOf, OpSpec, RoundingSchedule, StateInvalidation

SITES = ["trainer_fwd", "trainer_score", "engine_prefill", "engine_decode"]
ENGINE = ["engine_prefill", "engine_decode"]
GFX950 = frozenset({"gfx950"})


def register(reg) -> None:
    reg.register_op(
        OpSpec(name="gdn.core", sites=list(SITES)).add_impl(
            ImplSpec(
                impl_id="hip_fused_recurrent",
                version=1,
                supported_archs=GFX950,
                rounding=RoundingSchedule(
                    machine_assertable={
                        "kernel": OneOf("recurrent", "cpr"),
                        "state_dtype": "fp32",
                        "cpr": "entry chain fp32 per chunk boundary; running state = chain rounded to the wire dtype "
                               "at each boundary; chunk 64",
                        "recurrence": "token-level: S*=exp(g); v-=S.k; v*=beta; S+=k (x) v; o=S.q",
                        "dot": "8 state floats per lane as two fma chains (even, odd k), then lane tree",
                        "fma": "explicit only",
                        "time_tile": "staging only; never changes a value",
                    },
                    documentary=(
                        "The gated delta rule evaluated token by token with the fp32 state held in "
                        "registers. Prefill, chunked prefill and decode run the same recurrence, so a "
                        "sequence's outputs and final state do not depend on how it was cut into calls."
                    ),
                ),
                capabilities={"prefill_equals_decode": True},
                subsumes=("gdn.l2norm", "gdn.gating"),
                hazards=["null_lanes", "t_zero", "non_contiguous"],
            )
        )
    )
    reg.register_op(
        OpSpec(name="gdn.l2norm", sites=list(SITES)).add_impl(
            ImplSpec(
                impl_id="hip_l2norm",
                version=1,
                supported_archs=GFX950,
                rounding=RoundingSchedule(
                    machine_assertable={"eps": 1e-6, "rsqrt": "1/sqrtf", "sum": "8-wide tree then lane tree"},
                    documentary="x / sqrt(sum(x^2) + eps) per head, in fp32, rounded once to the io dtype.",
                ),
            )
        )
    )
    reg.register_op(
        OpSpec(name="gdn.gating", sites=list(SITES)).add_impl(
            ImplSpec(
                impl_id="hip_gate",
                version=1,
                supported_archs=GFX950,
                rounding=RoundingSchedule(
                    machine_assertable={"softplus_threshold": 20, "g": "-exp(A_log) * softplus(a + dt_bias)", "beta": "sigmoid(b)"},
                    documentary="The decay g and the write strength beta of the delta rule, elementwise in fp32.",
                ),
            )
        )
    )
    reg.register_op(
        OpSpec(name="gdn.conv", sites=list(SITES)).add_impl(
            ImplSpec(
                impl_id="hip_causal_conv",
                version=1,
                supported_archs=GFX950,
                rounding=RoundingSchedule(
                    machine_assertable={
                        "accumulate": "fp32, taps oldest to newest, bias first",
                        "activation": "silu",
                        "forms": "packed prefill and single-token update are the same per-token sum",
                    },
                    documentary=(
                        "Depthwise causal convolution over packed sequences with a carried state of W-1 "
                        "tokens. The update form is the prefill form at T=1, so the two agree bitwise."
                    ),
                ),
                hazards=["t_zero", "null_lanes"],
            )
        )
    )
    reg.register_op(
        OpSpec(name="gdn.state", sites=list(ENGINE)).add_impl(
            ImplSpec(
                impl_id="hip_private_pool",
                version=1,
                supported_archs=GFX950,
                rounding=RoundingSchedule(
                    machine_assertable={"ssm_cache_dtype": OneOf("float32"), "null_row": 0},
                    documentary=(
                        "Recurrent and convolution state live in pools owned by the layer, one row per "
                        "live request; row 0 is the null row that padded lanes read and never write."
                    ),
                ),
                state_invalidation=StateInvalidation(
                    condition="weight_sync or sleep_wake: every row is released and zeroed before the next forward"
                ),
                hazards=["null_lanes"],
            )
        )
    )

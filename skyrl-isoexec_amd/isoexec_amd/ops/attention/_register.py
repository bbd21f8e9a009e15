"""Registry entry for attention (reference: isoexec/ops/attention/_register.py)."""

from ...core.registry import ImplSpec, OpSpec, RoundingSchedule

SITES = ["trainer_fwd", "trainer_score", "engine_prefill", "engine_decode"]


def register(reg) -> None:
    reg.register_op(
        OpSpec(name="attention.varlen", sites=list(SITES)).add_impl(
            ImplSpec(
                impl_id="hip_varlen_ns1",
                version=1,
                supported_archs=frozenset({"gfx950"}),
                rounding=RoundingSchedule(
                    machine_assertable={
                        "num_splits": 1,
                        "window_size": [-1, 0],
                        "key_block": 32,
                        "scores": "v_mfma_f32_32x32x16_bf16 over d in 8 steps, fp32, then * scale",
                        "softmax": "online, per block: max, exp2((s-m)*log2e), l = l*a + (lo+hi)",
                        "pv": "bf16(p) x v by MFMA, fp32 accumulate, rescaled by a per block",
                        "output_round": "bf16(O / l)",
                    },
                    documentary=(
                        "Every query walks the keys of its own sequence in blocks of 32 from position 0 "
                        "to its own position, one walk, no split. A block past a query's position leaves "
                        "its accumulators bit-identical, so the packed full-sequence call, a chunked "
                        "prefill and a one-token decode step give the same bits for the same query."
                    ),
                ),
                capabilities={"query_length_invariant": True},
                hazards=["non_contiguous", "null_lanes"],
            )
        )
    )

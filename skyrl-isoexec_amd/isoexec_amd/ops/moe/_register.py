"""Registry entries for the mixture-of-experts family (reference: isoexec/ops/moe/_register.py)."""

from ...core.registry import PER_MODEL, ImplSpec, OneOf, OpSpec, RoundingSchedule

SITES = ["trainer_fwd", "trainer_score", "engine_prefill", "engine_decode"]
GFX950 = frozenset({"gfx950"})


def register(reg) -> None:
    reg.register_op(
        OpSpec(name="moe.router", sites=list(SITES)).add_impl(
            ImplSpec(
                impl_id="hip_fused_topk",
                version=1,
                supported_archs=GFX950,
                rounding=RoundingSchedule(
                    machine_assertable={
                        "logits": "fp32 GEMM, v_mfma_f32_32x32x2_f32, K left to right",
                        "score": OneOf("softmax_then_topk", "topk_then_softmax"),
                        "ties": "lowest expert index wins",
                        "topk": PER_MODEL,
                        "experts": PER_MODEL,
                    },
                    documentary=(
                        "One wave per token: softmax over the expert logits in fp32, top-k by repeated "
                        "arg-max with ties to the lowest index, optional renormalisation. Per-token work "
                        "only, so membership and weights do not depend on the batch."
                    ),
                ),
                hazards=["tie_boundaries", "e_mismatch"],
            )
        )
    )
    reg.register_op(
        OpSpec(name="moe.dispatch", sites=list(SITES)).add_impl(
            ImplSpec(
                impl_id="hip_bitmask_index",
                version=1,
                supported_archs=GFX950,
                rounding=RoundingSchedule(
                    machine_assertable={"order": "expert-major, token-ascending inside an expert", "arithmetic": "integer"},
                    documentary="The permutation is built from per-expert token bitmasks and popcounts; no value is rounded.",
                ),
                hazards=["t_zero"],
            )
        )
    )
    reg.register_op(
        OpSpec(name="moe.experts", sites=list(SITES)).add_impl(
            ImplSpec(
                impl_id="hip_grouped_mfma",
                version=1,
                supported_archs=GFX950,
                rounding=RoundingSchedule(
                    machine_assertable={
                        "gemm": "same K order as op mm",
                        "epilogue": "bf16(gate) -> bf16(silu) -> bf16(* up) -> bf16(* prob)",
                        "split_k": 1,
                    },
                    documentary=(
                        "Grouped SwiGLU: fc1 over gathered rows with the gate and up rows interleaved, the "
                        "activation in the epilogue, then fc2. A row's value depends on its own token and "
                        "expert only, never on the tile it landed in."
                    ),
                ),
                capabilities={"batch_invariant": True},
                hazards=["e_mismatch", "t_zero"],
            )
        )
    )
    reg.register_op(
        OpSpec(name="moe.combine", sites=list(SITES)).add_impl(
            ImplSpec(
                impl_id="hip_fixed_order",
                version=1,
                supported_archs=GFX950,
                rounding=RoundingSchedule(
                    machine_assertable={"order": "a token's k slots by ascending expert index", "leaf_dtype": OneOf("fp32", "bf16")},
                    documentary="Each token sums its k expert rows in a fixed order; no atomics.",
                ),
            )
        )
    )

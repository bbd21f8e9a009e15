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
                subsumes=("moe.blockmap",),
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
                subsumes=("moe.epilogue", "moe.weights"),
                hazards=["e_mismatch", "t_zero"],
            )
        )
    )
    # The three ops below are separate, engine-only fusions in the reference (ops/moe/_register.py:483-604). Here each
    # is how the op above it works at every site, so the impls above absorb them; they are registered so that the
    # vocabulary of ops is the reference's and a contract can name what absorbed them.
    reg.register_op(
        OpSpec(name="moe.blockmap", sites=list(SITES)).add_impl(
            ImplSpec(
                impl_id="hip_in_dispatch",
                version=1,
                supported_archs=GFX950,
                rounding=RoundingSchedule(
                    machine_assertable={
                        "integer_only": True,
                        "outputs": ["tile_expert", "tile_row0", "tile_nrows", "n_tiles"],
                        "shape_static": True,  # bound ceil(T k / BM) + E known on the host; later tiles exit on the device count
                        "launches": "inside the permutation (one launch for a batch of at most 256 tokens)",
                    },
                    documentary="The row-tile map of the grouped GEMMs, written by the permutation's offsets step; integers only.",
                ),
                capabilities={"hip_graph": True},
                hazards=["e_mismatch", "null_lanes"],
            )
        )
    )
    reg.register_op(
        OpSpec(name="moe.epilogue", sites=list(SITES)).add_impl(
            ImplSpec(
                impl_id="hip_fused_swiglu",
                version=1,
                supported_archs=GFX950,
                rounding=RoundingSchedule(
                    machine_assertable={
                        "folded_into": "fc1_gemm_epilogue",
                        "gate_and_up_in_one_wave": True,  # weight rows interleaved so a wave holds a gate tile and its up tile
                        "intermediate_materialized": False,  # the [T k, 2f] gate/up product never reaches memory
                        "chain": "bf16(gate) -> bf16(silu) -> bf16(* up) -> bf16(* prob)",
                    },
                    documentary="SwiGLU and the routing weight applied to the fc1 accumulators before the single store; elementwise, no reduction.",
                ),
                capabilities={"hip_graph": True},
                hazards=["non_contiguous"],
            )
        )
    )
    reg.register_op(
        OpSpec(name="moe.weights", sites=list(SITES)).add_impl(
            ImplSpec(
                impl_id="single_buffer",
                version=1,
                supported_archs=GFX950,
                rounding=RoundingSchedule(
                    machine_assertable={"buffer_shape": "[E, *param_shape]", "single_storage": True, "per_forward_copy": False},
                    documentary="The experts' weights are one [E, ...] tensor per role that the grouped GEMMs index by expert; nothing is stacked per forward.",
                ),
                capabilities={"hip_graph": True},
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

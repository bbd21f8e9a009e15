"""Registry entries for the token log-probability (reference: isoexec/ops/logprobs/_register.py)."""

from ...core.registry import PER_MODEL, ImplSpec, OpSpec, RoundingSchedule

SITES = ["trainer_fwd", "trainer_score", "engine_prefill", "engine_decode"]
GFX950 = frozenset({"gfx950"})


def register(reg) -> None:
    reg.register_op(
        OpSpec(name="logprobs.log_softmax", sites=list(SITES)).add_impl(
            ImplSpec(
                impl_id="hip_rowinv_leaftree",
                version=1,
                supported_archs=GFX950,
                rounding=RoundingSchedule(
                    machine_assertable={
                        "compute_dtype": "fp32",
                        "leaves": PER_MODEL,
                        "block": 4096,
                        "accum": "kahan_fp32",
                        "block_sum": "512 column sums over 8 chunks left to right, then adjacent-pairwise tree",
                        "exp": "exp2((x - m) * log2(e)) by the hardware exp2",
                        "reduction": [
                            "amax", "sub", "exp", "leaf_kahan_sum", "leaf_tree_combine", "log", "gather", "sub", "sub",
                        ],
                        "leaf_boundaries": "V/G fixed",
                        "combine": "combine_order(G)",
                        "launch_shapes": "row-per-workgroup and split-row compute identical bits",
                    },
                    documentary=(
                        "logprob = (x_target - m) - log(S): m is the exact row maximum, S is assembled "
                        "from G fixed contiguous vocabulary leaves (Kahan fp32 sums over blocks of 4096) "
                        "combined by the combine_order(G) tree. Nothing depends on the number of rows in "
                        "the call or on which launch shape ran, so a trainer's [B*S, V] call and an "
                        "engine's sampled-rows call give the same bits for the same row."
                    ),
                ),
                capabilities={"row_count_invariant": True, "tp_invariant": True},
                hazards=["subnormals", "non_contiguous"],
            )
        )
    )
    reg.register_op(
        OpSpec(name="logprobs.lm_head_slice", sites=["engine_prefill", "engine_decode"]).add_impl(
            ImplSpec(
                impl_id="sampled_rows",
                version=1,
                supported_archs=GFX950,
                rounding=RoundingSchedule(
                    machine_assertable={"rows": "sampled_only", "gather_output": True},
                    documentary=(
                        "The output layer is applied to the sampled rows only. Pure row selection: the "
                        "GEMM and the log-softmax are row-invariant, so the selected rows keep their bits."
                    ),
                ),
                capabilities={"split_lm_head": True},
            )
        )
    )

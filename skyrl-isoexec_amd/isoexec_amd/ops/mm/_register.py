"""Registry entries for the dense GEMM (reference: isoexec/ops/mm/_register.py).

One implementation serves all four sites: the kernel's reduction order over K depends on K alone, so
a row's value does not depend on how many rows share the launch or which tile shape ran it.
"""

from ...core.registry import ImplSpec, OneOf, OpSpec, RoundingSchedule

SITES = ["trainer_fwd", "trainer_score", "engine_prefill", "engine_decode"]
GFX950 = frozenset({"gfx950"})


def register(reg) -> None:
    reg.register_op(
        OpSpec(name="mm", sites=list(SITES)).add_impl(
            ImplSpec(
                impl_id="hip_mfma_batch_invariant",
                version=1,
                supported_archs=GFX950,
                rounding=RoundingSchedule(
                    machine_assertable={
                        "operands": "bf16",
                        "accumulate": "fp32",
                        "instruction": "v_mfma_f32_32x32x16_bf16",
                        "k_tile": 64,
                        "split_k": 1,
                        # One accumulator per output element walks K in tiles of 64; inside a tile the
                        # four MFMA steps take 16-wide chunks (s, 4+s) for the two lane halves.
                        "k_order": "tile-major, mfma step s reads chunks (s, 4+s)",
                        "output_round": "one fp32->bf16 round-to-nearest-even after bias",
                        "tile": OneOf("auto", "32x256", "128x128", "128x256", "256x256"),
                    },
                    documentary=(
                        "C = A @ W^T with bf16 operands and a single fp32 accumulator per element, no "
                        "split-K and no floating-point atomics. Every tile shape walks K in the same "
                        "order, so the result is independent of M, of the tile chosen and of the "
                        "position of a row inside the launch."
                    ),
                ),
                capabilities={"batch_invariant": True, "row_max_epilogue": True},
                hazards=["non_contiguous", "profiling_shapes"],
            )
        )
    )

"""bench.py sorts the kernels of a profiled step into the parts of a layer by the order of their launch."""
import os
import sys

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), ".."))
import bench  # noqa: E402


def test_kernels_of_a_step_are_sorted_into_the_parts_of_a_layer():
    decode_layer = ["add_stack_rmsnorm_kernel<bf16>", "gemm_rows_kernel<1, 2, 2, 4, 4, 0, float>", "qk_prep_kernel<bf16>",
                    "attn_mfma_kernel<1, 128, true>", "attn_merge_kernel", "gemm_rows_kernel<1, 1, 4, 4, 4, 0, float>",
                    "add_stack_rmsnorm_kernel<bf16>", "gemm_rows_kernel<1, 8, 1, 4, 4, 1, arle::bf16>",
                    "gemm_rows_kernel<1, 1, 4, 4, 4, 0, float>"]
    library_layer = ["rmsnorm_vec_kernel", "Cijk_Alik_Bljk_BBS_MT256", "qk_prep_bf16x8_kernel", "attn_prefill_plan_kernel",
                     "attn_prefill_dma_kernel<false>", "Cijk_Alik_Bljk_BBS_MT160", "rmsnorm_vec_kernel",
                     "Cijk_Alik_Bljk_BBS_MT256", "silu_mul_bf16x8_kernel", "gemm_stream_kernel<4, 8, 4, float>",
                     "sum_partials_kernel"]
    names = (["embed_gather_kernel"] + decode_layer + library_layer
             + ["add_stack_rmsnorm_kernel<float>", "gemm_rows_kernel<1, 8, 1, 4, 4, 0, float>", "argmax_chunks_kernel"])
    want = (["other"] + ["norm", "qkv", "qk_prep", "attention", "attention", "o", "norm", "gate_up", "down"]
            + ["norm", "qkv", "qk_prep", "attention", "attention", "o", "norm", "gate_up", "gate_up", "down", "down"]
            + ["norm", "head", "other"])
    assert bench.classify_step(names, layers=2) == want
    tiles = ["rmsnorm", "Cijk_a", "qk_prep", "attn_prefill_lds_kernel<128>", "Cijk_b", "rmsnorm",
             "gemm_tiles_kernel<4, 2, 4, 4, false, 1, arle::bf16>", "Cijk_c", "rmsnorm", "Cijk_head"]
    assert bench.classify_step(tiles, layers=1) == ["norm", "qkv", "qk_prep", "attention", "o", "norm", "gate_up", "down",
                                                    "norm", "head"]
    # single decoded tokens: no preparation kernel, the attention's kernel is the first behind the q|k|v product
    folded = ["embed_gather_kernel", "rmsnorm", "gemm_rows_kernel<1, 2, 2, 4, 4, 0, float>", "attn_mfma_kernel<1, 128, true, true>",
              "attn_merge_kernel", "gemm_rows_kernel<1, 1, 4, 4, 4, 0, float>", "add_stack_rmsnorm_kernel<bf16>",
              "gemm_rows_kernel<1, 8, 1, 4, 4, 1, arle::bf16>", "gemm_rows_kernel<1, 1, 4, 4, 4, 0, float>", "rmsnorm", "Cijk_head"]
    assert bench.classify_step(folded, layers=1) == ["other", "norm", "qkv", "attention", "attention", "o", "norm", "gate_up",
                                                     "down", "norm", "head"]
    assert bench.part_times([[(n, 1.0) for n in folded]], layers=1)["attention"] == 2.0


def test_a_step_whose_kernels_are_not_all_sorted_is_refused():
    """A kernel whose name no longer says what the sorting reads from it (here: an activation that never ends
    gate|up, so that down and the head stay empty) must not end up as figures in the record."""
    import pytest

    layer = ["rmsnorm", "Cijk_a", "qk_prep", "attn_prefill_dma_kernel<false, 1>", "Cijk_b", "rmsnorm",
             "gemm_tiles_kernel<4, 2, 4, 4, false, 7, arle::bf16>", "Cijk_c"]
    step = [("embed_gather_kernel", 1.0)] + [(n, 2.0) for n in layer] + [("rmsnorm", 1.0), ("Cijk_head", 3.0)]
    with pytest.raises(RuntimeError, match="down"):
        bench.part_times([step], layers=1)
    good = [(n.replace("false, 7", "false, 1"), us) for n, us in step]
    times = bench.part_times([good], layers=1)
    assert times["down"] == 2.0 and times["head"] == 3.0 and times["gate_up"] == 2.0 and times["kernels"] == len(good)


def test_bytes_and_flops_of_the_parts_add_up_to_the_step():
    c = bench.QWEN3_4B
    by_part = bench.part_bytes_decode(c, 8, 2064.0)
    whole = bench.decode_bytes(c, 8, 2064.0)
    assert 0.999 < sum(by_part.values()) / whole <= 1.0           # the rest: norm weights
    assert by_part["attention"] == 8 * 2064 * 147456
    flops = bench.part_flops_prefill(c, 2048)
    assert abs(sum(flops.values()) / bench.prefill_flops(c, 2048) - 1.0) < 1e-9

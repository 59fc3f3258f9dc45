#!/usr/bin/env python3
"""Regenerate the op descriptions (*.info) of this directory.

`c1`..`c5` are the five fused-operator configurations the backend is measured on; the `small_*` files are the same
patterns at sizes a scalar CPU run finishes instantly, plus ragged shapes that exercise tail handling.
Run from the repository root: python akg_amd/fixtures/make_fixtures.py
"""
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from akg_amd import op_desc  # noqa: E402

FIXTURES = {
    # measured configurations
    "c1_ew_tanh_add_mul_f32_1024x4096": lambda n: op_desc.elementwise_tanh_add_mul(1024, 4096, n),
    "c2_softmax_f16_8192x4096": lambda n: op_desc.softmax_last_axis(8192, 4096, "float16", n),
    "c3_layernorm_residual_bf16_16384x4096": lambda n: op_desc.layernorm_residual(16384, 4096, "bfloat16", 1e-5, n),
    "c4_quant_int8_residual_bf16_32768x8192": lambda n: op_desc.quant_int8_residual(32768, 8192, "bfloat16", n),
    "c5_gemm_i8_dequant_bias_gelu_4096x8192x8192": lambda n: op_desc.gemm_int8_dequant_bias_gelu(4096, 8192, 8192, "bfloat16", False, n),
    # plain streaming kernel of known size, used to calibrate the HBM traffic counters
    "calib_neg_f32_16384x4096": lambda n: _neg(16384, 4096, n),
    # streaming kernels with next to no arithmetic, of exactly the tensor sizes of c1 (3 reads + 1 write) and c2 (1 + 1)
    "calib_add3_f32_1024x4096": lambda n: _add3(1024, 4096, n),
    "calib_neg_f16_8192x4096": lambda n: _neg(8192, 4096, n, "float16"),
    # the sample of c5 the CPU baseline runs: 64 of the 4096 rows of A against the whole of B
    "c5_mslice64_gemm_i8_dequant_bias_gelu_64x8192x8192": lambda n: op_desc.gemm_int8_dequant_bias_gelu(64, 8192, 8192, "bfloat16", False, n),
    # small parity cases
    "small_ew_tanh_add_mul_f32_8x128": lambda n: op_desc.elementwise_tanh_add_mul(8, 128, n),
    "small_ew_tanh_add_mul_f32_7x33": lambda n: op_desc.elementwise_tanh_add_mul(7, 33, n),
    "small_softmax_f16_64x4096": lambda n: op_desc.softmax_last_axis(64, 4096, "float16", n),
    "small_softmax_f16_33x1000": lambda n: op_desc.softmax_last_axis(33, 1000, "float16", n),
    "small_softmax_f32_5x77": lambda n: op_desc.softmax_last_axis(5, 77, "float32", n),
    "small_layernorm_residual_bf16_64x4096": lambda n: op_desc.layernorm_residual(64, 4096, "bfloat16", 1e-5, n),
    "small_layernorm_residual_bf16_19x520": lambda n: op_desc.layernorm_residual(19, 520, "bfloat16", 1e-5, n),
    "small_quant_int8_residual_bf16_64x8192": lambda n: op_desc.quant_int8_residual(64, 8192, "bfloat16", n),
    "small_quant_int8_residual_bf16_37x1544": lambda n: op_desc.quant_int8_residual(37, 1544, "bfloat16", n),
    # rows that are not a power of two of chunks (3, 5 and 6 chunks per thread) and rows too long for registers
    # (walked in groups, once per reduction and once for the outputs; ragged last group)
    "small_softmax_f16_9x768": lambda n: op_desc.softmax_last_axis(9, 768, "float16", n),
    "small_layernorm_residual_bf16_5x5120": lambda n: op_desc.layernorm_residual(5, 5120, "bfloat16", 1e-5, n),
    "small_layernorm_residual_bf16_3x11008": lambda n: op_desc.layernorm_residual(3, 11008, "bfloat16", 1e-5, n),
    # rows that are not a multiple of the 16-byte chunk: element-aligned full-width accesses, overlapping last chunk
    "small_softmax_f16_7x4095": lambda n: op_desc.softmax_last_axis(7, 4095, "float16", n),
    "small_layernorm_residual_bf16_4x1001": lambda n: op_desc.layernorm_residual(4, 1001, "bfloat16", 1e-5, n),
    "small_quant_int8_residual_bf16_3x2051": lambda n: op_desc.quant_int8_residual(3, 2051, "bfloat16", n),
    "small_softmax_f16_3x70000": lambda n: op_desc.softmax_last_axis(3, 70000, "float16", n),
    "small_softmax_f32_2x50257": lambda n: op_desc.softmax_last_axis(2, 50257, "float32", n),
    "small_layernorm_residual_bf16_2x57000": lambda n: op_desc.layernorm_residual(2, 57000, "bfloat16", 1e-5, n),
    "small_layernorm_residual_bf16_2x66000": lambda n: op_desc.layernorm_residual(2, 66000, "bfloat16", 1e-5, n),
    "small_quant_int8_residual_bf16_2x131080": lambda n: op_desc.quant_int8_residual(2, 131080, "bfloat16", n),
    "small_gemm_i8_dequant_bias_gelu_256x512x256": lambda n: op_desc.gemm_int8_dequant_bias_gelu(256, 512, 256, "bfloat16", False, n),
    "small_gemm_i8_dequant_bias_gelu_256x512x256_tb": lambda n: op_desc.gemm_int8_dequant_bias_gelu(256, 512, 256, "bfloat16", True, n),
    "small_momentum_update_f32_37x130": lambda n: op_desc.momentum_update(37, 130, "float32", name=n),
    "small_momentum_update_bf16_64x256": lambda n: op_desc.momentum_update(64, 256, "bfloat16", name=n),
    "small_elemany_greater_f32_9x130": lambda n: op_desc.any_greater(9, 130, 2.5, "ElemAny", n),
    # op-table rows outside the measured fusions, one kernel per group
    "small_optable_unary_math_f32_37x130": lambda n: op_desc.optable_unary_math(37, 130, "float32", n),
    "small_optable_unary_math_f16_16x256": lambda n: op_desc.optable_unary_math(16, 256, "float16", n),
    "small_optable_predicates_logic_33x100": lambda n: op_desc.optable_predicates_logic(33, 100, n),
    "small_optable_pow_atan2_addn_f32_19x264": lambda n: op_desc.optable_pow_atan2_addn(19, 264, "float32", n),
    "small_optable_pow_atan2_addn_bf16_8x1024": lambda n: op_desc.optable_pow_atan2_addn(8, 1024, "bfloat16", n),
    "small_optable_int_div_21x77": lambda n: op_desc.optable_int_div(21, 77, n),
    # MatMul in the reference's own arithmetic: a 16-bit declared result (product and sum rounded to it at every k), and
    # shapes / element types the MFMA kernels do not take
    "small_gemm_f16_result_f16_bias_relu_70x200x36": lambda n: op_desc.gemm_bias_act(70, 200, 36, "float16", "relu", False, "float16", n),
    "small_gemm_bf16_result_bf16_bias_none_33x129x5_tb": lambda n: op_desc.gemm_bias_act(33, 129, 5, "bfloat16", "none", True, "bfloat16", n),
    "small_gemm_f32_bias_gelu_70x100x36": lambda n: op_desc.gemm_bias_act(70, 100, 36, "float32", "gelu", False, "float32", n),
    "small_gemm_bf16_bias_gelu_65x30x10": lambda n: op_desc.gemm_bias_act(65, 30, 10, "bfloat16", "gelu", False, "float32", n),
    # streaming reductions: direction Y, direction ALL, long rows, multi-output
    "small_reducey_sqsum_f32_1x5100x3072": lambda n: op_desc.square_reduce([1, 5100, 3072], [1], "float32", True, "ReduceSum", n),
    "small_reducey_sqsum_f32_3x37x50": lambda n: op_desc.square_reduce([3, 37, 50], [1], "float32", False, "ReduceSum", n),
    "small_reducey_max_f16_130x66": lambda n: op_desc.square_reduce([130, 66], [0], "float16", False, "ReduceMax", n),
    "small_reduceall_sqsum_f32_768x512": lambda n: op_desc.square_reduce([768, 512], [0, 1], "float32", False, "ReduceSum", n),
    "small_reduceall_min_f32_7x333": lambda n: op_desc.square_reduce([7, 333], [0, 1], "float32", False, "ReduceMin", n),
    "small_reducex_long_sqsum_f32_3x300000": lambda n: op_desc.square_reduce([3, 300000], [1], "float32", False, "ReduceSum", n),
    # rows and runs that are long and no multiple of the chunk: walked in chunk slots, the last one of a run overlapping
    "small_reducex_long_sqsum_f16_5x40001": lambda n: op_desc.square_reduce([5, 40001], [1], "float16", False, "ReduceSum", n),
    "small_bnstats_bf16_4x6x35x35": lambda n: op_desc.batchnorm_stats(4, 6, 35, 35, "bfloat16", n),
    # kept axes between reduced ones: batch-norm statistics (contiguous runs of H*W), and a [4,5,6,16] sum over axes 0, 2
    "small_bnstats_bf16_8x6x7x12": lambda n: op_desc.batchnorm_stats(8, 6, 7, 12, "bfloat16", n),
    "small_bnstats_update_bf16_8x6x7x12": lambda n: op_desc.batchnorm_stats_update(8, 6, 7, 12, "bfloat16", 0.9, n),
    "small_bnstats_update_f32_32x16x28x28": lambda n: op_desc.batchnorm_stats_update(32, 16, 28, 28, "float32", 0.9, n),
    "small_bnstats_f32_32x16x28x28": lambda n: op_desc.batchnorm_stats(32, 16, 28, 28, "float32", n),
    "small_reducey_sqsum_f32_4x5x6x16_axes02": lambda n: op_desc.square_reduce([4, 5, 6, 16], [0, 2], "float32", False, "ReduceSum", n),
    "small_reducey_max_f16_3x4x50x9_axes02_keep": lambda n: op_desc.square_reduce([3, 4, 50, 9], [0, 2], "float16", True, "ReduceMax", n),
    "small_biasgrad_bf16_2048x1024": lambda n: op_desc.bias_grad(2048, 1024, "bfloat16", n),
    "small_biasgrad_bf16_1000x4095": lambda n: op_desc.bias_grad(1000, 4095, "bfloat16", n),
    "small_biasgrad_f32_100x37": lambda n: op_desc.bias_grad(100, 37, "float32", n),
    "small_sub_exp_reducesum_split_f32_4x96x160": lambda n: op_desc.sub_exp_reduce_y(4, 96, 160, "float32", n),
    "small_mean_absmax_all_f32_1000x1000": lambda n: op_desc.mean_absmax_all(1000, 1000, "float32", n),
    # data-movement ops (indexed family)
    "small_view_chain_f32": lambda n: op_desc.view_chain(n),
    "small_transpose_bias_add_bf16_3x20x36": lambda n: op_desc.transpose_bias_add(3, 20, 36, "bfloat16", n),
    "small_transpose_0213_neg_f16_2x5x6x8": lambda n: op_desc.transpose_0213_neg([2, 5, 6, 8], "float16", n),
    "small_slice_concat_pad_add_i32": lambda n: op_desc.slice_concat_int(n),
    "small_transpose_reshape_add_f32_4x6x10": lambda n: op_desc.transpose_reshape_add(n),
    "small_transpose_bias_add_f32_2x100x200": lambda n: op_desc.transpose_bias_add(2, 100, 200, "float32", n),
    "small_transpose_sum_f32_2x70x3x80_perm0321": lambda n: op_desc.transpose_sum([2, 70, 3, 80], [0, 3, 2, 1], "float32", n),
    "small_transpose_sum_f16_130x66_perm10": lambda n: op_desc.transpose_sum([130, 66], [1, 0], "float16", n),
    "small_split_swiglu_bf16_37x264": lambda n: op_desc.split_swiglu(37, 264, "bfloat16", n),
    "small_split_swiglu_f32_5x9": lambda n: op_desc.split_swiglu(5, 9, "float32", n),
    # ArgMax over the innermost axis (row family: max, then the least position that holds it)
    "small_argmax_f32_37x1000": lambda n: op_desc.argmax_last_axis([37, 1000], "float32", False, "int32", None, n),
    "small_argmax_f16_3x5x333_keep_i64": lambda n: op_desc.argmax_last_axis([3, 5, 333], "float16", True, "int64", None, n),
    "small_argmax_bf16_scaled_4x70000": lambda n: op_desc.argmax_last_axis([4, 70000], "bfloat16", False, "int32", 0.5, n),
    "small_embedding_lookup_bf16_1000x96_ids5x33": lambda n: op_desc.embedding_lookup_scale(1000, 96, 5, 33, "bfloat16", n),
    "small_embedding_lookup_f32_50x7_ids3x4": lambda n: op_desc.embedding_lookup_scale(50, 7, 3, 4, "float32", n),
    # UnsortedSegmentSum (segment_sum family): short slices, a wide slice tiled over workgroups, 16-bit accumulation
    "small_segment_sum_f32_700x3_by_1x3_seg50": lambda n: op_desc.unsorted_segment_sum([700, 3], [1, 3], 50, "float32", "int32", n),
    "small_segment_sum_f32_300_by_10000_seg7": lambda n: op_desc.unsorted_segment_sum([300], [10000], 7, "float32", "int64", n),
    "small_segment_sum_bf16_4096_by_200_seg1000": lambda n: op_desc.unsorted_segment_sum([4096], [200], 1000, "bfloat16", "int32", n),
    "small_segment_sum_i32_1000_by_65_seg3": lambda n: op_desc.unsorted_segment_sum([1000], [65], 3, "int32", "int32", n),
    # descriptions no single kernel serves: run as a sequence of kernels cut at the reduction results
    "small_staged_softmax_f32_32x12x24x40_axis1": lambda n: op_desc.softmax_over_axis([32, 12, 24, 40], 1, "float32", n),
    "small_staged_softmax_f16_50x3000_axis0": lambda n: op_desc.softmax_over_axis([50, 3000], 0, "float16", n),
    "small_staged_bn_train_forward_f32_16x8x14x14": lambda n: op_desc.batchnorm_train_forward(16, 8, 14, 14, "float32", 1e-5, n),
    "small_staged_bn_train_forward_bf16_8x6x7x12": lambda n: op_desc.batchnorm_train_forward(8, 6, 7, 12, "bfloat16", 1e-5, n),
    "small_staged_layernorm_axis1_bf16_8x64x49": lambda n: op_desc.layernorm_over_axis1(8, 64, 49, "bfloat16", 1e-5, n),
    "small_staged_attention_probs_bf16_4x128x64x256": lambda n: op_desc.attention_probabilities(4, 128, 64, 256, "bfloat16", n),
    "small_staged_attention_probs_f16_3x40x64x136": lambda n: op_desc.attention_probabilities(3, 40, 64, 136, "float16", n),
    "small_staged_transposed_a_matmul_bf16_48x512x264": lambda n: op_desc.transposed_a_matmul_bias_relu(48, 512, 264, "bfloat16", n),
    "small_staged_transposed_a_matmul_f16_300x256x136": lambda n: op_desc.transposed_a_matmul_bias_relu(300, 256, 136, "float16", n),
    "small_sgdclip_update_f32_300x130": lambda n: op_desc.sgd_clip_by_global_norm(300, 130, "float32", 0.01, 1.0, n),
    "small_sgdclip_update_bf16_64x256": lambda n: op_desc.sgd_clip_by_global_norm(64, 256, "bfloat16", 0.01, 1.0, n),
    # many positions: grouped by segment first (short rows moved, wide rows through their positions)
    "small_segment_sum_f32_300000_by_3_seg5000": lambda n: op_desc.unsorted_segment_sum([300000], [3], 5000, "float32", "int32", n),
    "small_segment_sum_f16_150001_by_4_seg300": lambda n: op_desc.unsorted_segment_sum([150001], [4], 300, "float16", "int64", n),
    "small_segment_sum_f32_140000_by_40_seg129": lambda n: op_desc.unsorted_segment_sum([140000], [40], 129, "float32", "int32", n),
    "n3_transpose_bias_add_bf16_32x2048x1024": lambda n: op_desc.transpose_bias_add(32, 2048, 1024, "bfloat16", n),
    # float MatMul + bias + activation on the bfloat16 / float16 MFMA path
    "small_gemm_bf16_bias_gelu_256x512x256": lambda n: op_desc.gemm_bias_act(256, 512, 256, "bfloat16", "gelu", False, "float32", n),
    "small_gemm_bf16_bias_gelu_256x512x256_tb": lambda n: op_desc.gemm_bias_act(256, 512, 256, "bfloat16", "gelu", True, "float32", n),
    "small_gemm_f16_bias_relu_200x264x136": lambda n: op_desc.gemm_bias_act(200, 264, 136, "float16", "relu", False, "float32", n),
    "small_gemm_f16_bias_relu_200x264x136_tb": lambda n: op_desc.gemm_bias_act(200, 264, 136, "float16", "relu", True, "float32", n),
    "small_gemm_bf16_bias_none_520x1024x776": lambda n: op_desc.gemm_bias_act(520, 1024, 776, "bfloat16", "none", False, "float32", n),
    # few tiles, long K: K split over several workgroups per tile (partials in the workspace, last one finishes)
    "small_gemm_i8_dequant_bias_gelu_64x4096x256": lambda n: op_desc.gemm_int8_dequant_bias_gelu(64, 4096, 256, "bfloat16", False, n),
    "small_gemm_i8_dequant_bias_gelu_300x2064x520_tb": lambda n: op_desc.gemm_int8_dequant_bias_gelu(300, 2064, 520, "bfloat16", True, n),
    "small_gemm_bf16_bias_gelu_100x2048x520": lambda n: op_desc.gemm_bias_act(100, 2048, 520, "bfloat16", "gelu", False, "float32", n),
    "small_gemm_f16_bias_relu_16x3000x264_tb": lambda n: op_desc.gemm_bias_act(16, 3000, 264, "float16", "relu", True, "float32", n),
    "small_batchmatmul_scale_mask_bf16_3x200x64x136_tb": lambda n: op_desc.batch_matmul_scale_mask(3, 200, 64, 136, "bfloat16", True, n),
    "small_batchmatmul_scale_mask_f16_2x256x128x256": lambda n: op_desc.batch_matmul_scale_mask(2, 256, 128, 256, "float16", False, n),
    "n2_gemm_bf16_bias_gelu_4096x8192x8192": lambda n: op_desc.gemm_bias_act(4096, 8192, 8192, "bfloat16", "gelu", False, "float32", n),
    # the next measured row: bias / scale gradients of a [16384, 4096] bf16 activation (two column sums in one pass)
    "n4_softmax_f16_512x131072": lambda n: op_desc.softmax_last_axis(512, 131072, "float16", n),
    "n5_bnstats_bf16_256x64x56x56": lambda n: op_desc.batchnorm_stats(256, 64, 56, 56, "bfloat16", n),
    "n6_gemm_bf16_bias_gelu_16x8192x8192": lambda n: op_desc.gemm_bias_act(16, 8192, 8192, "bfloat16", "gelu", False, "float32", n),
    "n1_biasgrad_bf16_16384x4096": lambda n: op_desc.bias_grad(16384, 4096, "bfloat16", n),
    # the shape of the reference's largest UnsortedSegmentSum description: 24.5 million positions of 3 floats into 4954 rows
    "n7_segment_sum_f32_4954x4953_by_1x3_seg4954": lambda n: op_desc.unsorted_segment_sum([4954, 4953], [1, 3], 4954, "float32", "int32", n),
    # reductions over an axis that is not the innermost one, whose results meet the tensor again (column kernel, or one
    # kernel per reduction level): a softmax over the 21 classes of a segmentation map, a channels-first LayerNorm
    "n8_softmax_axis1_f16_32x21x512x512": lambda n: op_desc.softmax_over_axis([32, 21, 512, 512], 1, "float16", n),
    "n9_layernorm_axis1_bf16_64x768x1024": lambda n: op_desc.layernorm_over_axis1(64, 768, 1024, "bfloat16", 1e-5, n),
}


def _neg(rows, cols, name, dtype="float32"):
    b = op_desc.DescBuilder(name)
    x = b.input([rows, cols], dtype)
    return b.dumps([b.unary("Neg", x)])


def _add3(rows, cols, name):
    b = op_desc.DescBuilder(name)
    x, y, z = [b.input([rows, cols], "float32") for _ in range(3)]
    return b.dumps([b.add(b.add(x, y), z)])


def main():
    for name, make in FIXTURES.items():
        path = os.path.join(HERE, name + ".info")
        with open(path, "w", encoding="utf-8") as f:
            f.write(make(name))
            f.write("\n")
        print("wrote", os.path.relpath(path))


if __name__ == "__main__":
    main()

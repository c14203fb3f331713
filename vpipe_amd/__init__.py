"""MI355X (gfx950) implementation of VPIPE's 4-bit / group-64 affine quantized
linear path: QMV, QMM (+ fused runtime LoRA), dense expansion and the packer.

The product is the C-ABI shared library `libvpq.so` (include/vpq.h).  This
package only loads it and hands it torch device pointers; it contains no CPU
implementation of any operator and raises if the library is missing.
"""
from . import capi  # noqa: F401
from .capi import (VpqError, argmax_bf16, argmax_bf16_static, dequant_w4g32, qmv_w4g32, qmm_dense_route_w4g32, dequant_w4g64, dequant_w8g64, qmv_w8g64, qmm_dense_route_w8g64, embed_gather_w4g64, f16_to_bf16, gather_down_qmv_w4g64, gather_qmv_gated_w4g64, linear_twin, qmm_w4g32, qmm_w8g64, qmm_grouped_gated_w8g64, qmm_grouped_down_w8g64, gather_qmv_gated_split, dequant_w4g64_f16, qmv_w4g64_f16, qmm_dense_route_w4g64_f16, qmm_w4g64_f16, qmm_lora_w4g64_f16, lora_a_f16, quantize, qmm_dense_route_lora, dequant_w8_f16, qmm_dense_route_w8_f16, qmv_gelu_mul_w4g64, qmv_gelu_mul_w8g64, qmv_gelu_mul_w4g32, requant_w8_to_w4, moe_gate_w8g64, qmv_group_w4g32, qmv_group_w8g64, rmsnorm_bf16, qmv_qkv_rms, dequant_w8g32, qmv_w8g32, qmm_dense_route_w8g32, qmv_group_w4g64_f16, gather_down_qmv_w8g64, gather_qmv_gated_w8g64, qmv_gated_w8g64, grouped_block_rows, moe_max_tiles, moe_sort_pairs, moe_scatter_back, qmm_grouped_down_w4g64, qmm_grouped_gated_w4g64, interleave_gate_up, lib_path, build_id, sample_topp_bf16, sample_hist_bf16, sample_hist_slabs, qmv_grouped_gated_w4g64, qmv_grouped_down_w4g64, qmv_grouped_gated_w8g64, qmv_grouped_down_w8g64, linear_swiglu_w4g64,  # noqa: F401
                   linear_w4g64, load, lora_a, qmm_dense_route_w4g64, qmm_splitk_w4g64, qmm_swiglu_w4g64, qmm_w4g64, qmv_group_w4g64,
                   qmv_swiglu_w4g64, qmv_w4g64, qmv_workspace, quantize_w4g64)

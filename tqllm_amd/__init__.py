"""MI355X-native mixture-of-experts layer with the operator interface of tqLLM's src/experts.

The product is the C-ABI HIP library libtqmoe.so (include/tqmoe.h); this package is the host-side mirror of the
reference's operator interface on top of it (torch supplies device memory and streams, nothing else).
"""
from .api import (BF16, F16, F32, IQ1_S, IQ2_S, IQ2_XS, IQ2_XXS, IQ3_XXS, Q2_K, Q3_K, Q4_0, GATE_SIGMOID, GATE_SOFTMAX, GATE_SOFTMAX_WEIGHT, GATE_SQRT_SOFTPLUS, IQ3_S, IQ4_NL, IQ4_XS, NVFP4G, Q4_K, Q5_K, Q6_K, Q8_0, ExpertBank, MoeLayer, TqmoeError, abi_version, add_rmsnorm, moe_combine_residual,  # noqa: F401
                  expert_down, expert_gateup, expert_gemm, expert_gemm_gateup, expert_gemm_gateup_i8, expert_gemm_i8, quant_rows_i8, group_rows_i8, gather_rows_i8, quant_rows_i8_blocks, group_rows_i8_blocks, gather_rows_i8_blocks, expert_gemm_gateup_i8_blocks, expert_gemm_i8_blocks, expert_gemm_gateup_fp8, expert_gemm_fp8, quant_rows_fp8, group_rows_fp8, expert_matvec, expert_matvec2, lib, moe_combine, moe_combine_strided, moe_dispatch, moe_dispatch_into, moe_extend_ids, moe_router, moe_swiglu, moe_topk, moe_topk2, quant_act, moe_group, moe_count, moe_dedup_maps, lists_from_groups, expert_gemm_i8_ref, expert_matvec_dedup)

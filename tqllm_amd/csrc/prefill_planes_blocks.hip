// The int8 grouped products with a scale per row and 32-value sub-block (the reference's per-32-block activation mode of
// expert_gemm_i8, src/formats/weight/quant_kernels.cuh:13-16, mode 1): the same kernel, every sub-block's integer sums
// scaled on their own.
#include "prefill_planes_kernels.cuh"

namespace tqmoe {

int32_t plane_gemm_blocks(uint32_t type, int nb, bool gateup, const GemmArgs & k, unsigned blocks, hipStream_t s) {
    switch (type) {
        case TQMOE_IQ4_XS: plane_gemm_launch<WIq4xsSub, true>(nb, gateup, k, blocks, s); break;
        case TQMOE_IQ3_S: plane_gemm_launch<WIq3s, true>(nb, gateup, k, blocks, s); break;
        case TQMOE_Q4_K: plane_gemm_launch<WQ4kSub, true>(nb, gateup, k, blocks, s); break;
        case TQMOE_IQ3_XXS: plane_gemm_launch<WIq3xxs, true>(nb, gateup, k, blocks, s); break;
        case TQMOE_IQ2_XXS: plane_gemm_launch<WIq2xxs, true>(nb, gateup, k, blocks, s); break;
        case TQMOE_IQ2_XS: plane_gemm_launch<WIq2xs, true>(nb, gateup, k, blocks, s); break;
        case TQMOE_IQ2_S: plane_gemm_launch<WIq2s, true>(nb, gateup, k, blocks, s); break;
        case TQMOE_IQ1_S: plane_gemm_launch<WIq1s, true>(nb, gateup, k, blocks, s); break;
        case TQMOE_IQ4_NL: plane_gemm_launch<WIq4nl, true>(nb, gateup, k, blocks, s); break;
        default: return -1;
    }
    return 0;
}

}  // namespace tqmoe

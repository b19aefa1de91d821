// The int8 grouped products of the older GGUF block formats with one scale per 32 weights (Q5_K, Q4_0, Q8_0), with a scale
// per row or per row and 32-value sub-block: the kernel of prefill_planes_kernels.cuh with their traits (a translation unit
// of its own so that it compiles beside the others).
#include "prefill_planes_kernels.cuh"

namespace tqmoe {

int32_t plane_gemm_legacy(uint32_t type, int nb, bool gateup, bool blk, const GemmArgs & k, unsigned blocks, hipStream_t s) {
    switch (type) {
        case TQMOE_Q5_K:
            if (blk) plane_gemm_launch<WQ5kSub, true>(nb, gateup, k, blocks, s);
            else plane_gemm_launch<WQ5k>(nb, gateup, k, blocks, s);
            break;
        case TQMOE_Q4_0:
            if (blk) plane_gemm_launch<WQ4_0, true>(nb, gateup, k, blocks, s);
            else plane_gemm_launch<WQ4_0>(nb, gateup, k, blocks, s);
            break;
        case TQMOE_Q8_0:
            if (blk) plane_gemm_launch<WQ8_0, true>(nb, gateup, k, blocks, s);
            else plane_gemm_launch<WQ8_0>(nb, gateup, k, blocks, s);
            break;
        default: return -1;
    }
    return 0;
}

}  // namespace tqmoe

// Entry helpers of the 8-bit grouped products: the row quantisers, the grouped operand and the per-row-scale products.
#include "prefill_planes_kernels.cuh"

namespace tqmoe {

// ---------------------------------------------------------------------------------------------- entry helpers
int64_t grouped_row_tiles(int64_t assignments, int experts) { return (assignments + 31) / 32 + experts; }

// f8: E4M3 bytes with scale amax / 448 in place of int8 bytes with scale amax / 127
int32_t enqueue_quant_rows_i8(const void * x, uint32_t xtype, int64_t rows, int cols, int8_t * q, float * scale, hipStream_t s, bool f8) {
    const unsigned blocks = unsigned((rows + 3) / 4);
#define TQMOE_QUANT(XT) (f8 ? quant_rows_k<XT, true><<<blocks, 256, 0, s>>>(x, rows, cols, q, scale) : quant_rows_k<XT, false><<<blocks, 256, 0, s>>>(x, rows, cols, q, scale))
    switch (xtype) {
        case TQMOE_F32: TQMOE_QUANT(TQMOE_F32); break;
        case TQMOE_F16: TQMOE_QUANT(TQMOE_F16); break;
        default: TQMOE_QUANT(TQMOE_BF16); break;
    }
#undef TQMOE_QUANT
    return 0;
}

// a scale per 32 values and, when qsum is given, the sums of q per 16 values
int32_t enqueue_quant_rows_i8_blocks(const void * x, uint32_t xtype, int64_t rows, int cols, int8_t * q, float * scale, int16_t * qsum, hipStream_t s) {
    const unsigned blocks = unsigned((rows + 3) / 4);
    switch (xtype) {
        case TQMOE_F32: quant_rows_k<TQMOE_F32, false, true><<<blocks, 256, 0, s>>>(x, rows, cols, q, scale, qsum); break;
        case TQMOE_F16: quant_rows_k<TQMOE_F16, false, true><<<blocks, 256, 0, s>>>(x, rows, cols, q, scale, qsum); break;
        default: quant_rows_k<TQMOE_BF16, false, true><<<blocks, 256, 0, s>>>(x, rows, cols, q, scale, qsum); break;
    }
    return 0;
}

int64_t grouped_scale_words(int64_t assignments, int experts) { return grouped_row_tiles(assignments, experts) * 32 + 3 * (int64_t(experts) + 1) + kPlanCounters; }

template <int XT, bool F8, bool BLK>
static void group_rows_launch(const void * x, int cols, const int * counts, const int * offsets, const int * perm, int experts, int64_t tiles, int xdiv, int8_t * q,
                              float * scale, const Plan & plan, hipStream_t s, float * block_scale) {
    if (cols % 256 == 0 && cols <= 2048) {
        const size_t lds = size_t(32) * size_t(cols + 16);
        auto launch = [&](auto kernel) {
            if (lds > 65536 - 1024) allow_dynamic_lds(reinterpret_cast<const void *>(kernel), 32 * (2048 + 16));
            kernel<<<unsigned(tiles), 256, lds, s>>>(x, cols, counts, offsets, perm, experts, xdiv, q, scale, plan, block_scale);
        };
        if (cols <= 512) launch(group_rows_tile_k<XT, 1, F8, BLK>);
        else if (cols <= 1024) launch(group_rows_tile_k<XT, 2, F8, BLK>);
        else if (cols <= 1536) launch(group_rows_tile_k<XT, 3, F8, BLK>);
        else launch(group_rows_tile_k<XT, 4, F8, BLK>);
        return;
    }
    group_rows_k<XT, F8, BLK><<<unsigned(tiles * 4), 256, 0, s>>>(x, cols, counts, offsets, perm, experts, xdiv, q, scale, plan, block_scale);
}

// block_scale (int8 only): a scale per row and 32-value block, [row tile][block][32 rows]; the rows' own scales are then 1
int32_t enqueue_group_rows_i8(const void * x, uint32_t xtype, int cols, const int * counts, const int * offsets, const int * perm, int experts,
                              int64_t assignments, int xdiv, int8_t * q, float * scale, hipStream_t s, bool f8, float * block_scale) {
    const int64_t tiles = grouped_row_tiles(assignments, experts);
    const Plan plan = plan_at(scale, tiles * 32, experts);
    plan_k<<<1, 64, 0, s>>>(counts, experts, plan);
#define TQMOE_GROUP(XT) (f8 ? group_rows_launch<XT, true, false>(x, cols, counts, offsets, perm, experts, tiles, xdiv, q, scale, plan, s, nullptr) \
                         : block_scale ? group_rows_launch<XT, false, true>(x, cols, counts, offsets, perm, experts, tiles, xdiv, q, scale, plan, s, block_scale) \
                                       : group_rows_launch<XT, false, false>(x, cols, counts, offsets, perm, experts, tiles, xdiv, q, scale, plan, s, nullptr))
    switch (xtype) {
        case TQMOE_F32: TQMOE_GROUP(TQMOE_F32); break;
        case TQMOE_F16: TQMOE_GROUP(TQMOE_F16); break;
        default: TQMOE_GROUP(TQMOE_BF16); break;
    }
#undef TQMOE_GROUP
    return 0;
}

int32_t enqueue_gather_rows_i8(const int8_t * rq, const float * rs, int cols, const int * counts, const int * offsets, const int * perm, int experts,
                               int64_t assignments, int xdiv, int8_t * q, float * scale, hipStream_t s, float * block_scale) {
    const int64_t tiles = grouped_row_tiles(assignments, experts);
    const Plan plan = plan_at(scale, tiles * 32, experts);
    plan_k<<<1, 64, 0, s>>>(counts, experts, plan);
    gather_rows_i8_k<<<unsigned(tiles), 256, 0, s>>>(rq, rs, cols, counts, offsets, perm, experts, xdiv, q, scale, plan, block_scale);
    return 0;
}

// bank formats with a plane GEMM: int8 operands (IQ4_XS, IQ4_NL, IQ3_S, IQ3_XXS, IQ2_XXS, IQ2_XS, IQ2_S, IQ1_S, Q4_K) or E4M3 operands (NVFP4G)
bool plane_gemm_has(uint32_t type) {
    return type == TQMOE_IQ4_XS || type == TQMOE_IQ3_S || type == TQMOE_Q4_K || type == TQMOE_NVFP4G || type == TQMOE_IQ3_XXS || type == TQMOE_IQ2_XXS ||
           type == TQMOE_IQ2_XS || type == TQMOE_IQ2_S || type == TQMOE_IQ1_S || type == TQMOE_IQ4_NL;
}
bool plane_gemm_is_fp8(uint32_t type) { return type == TQMOE_NVFP4G; }

// assignments = total entries of perm (it fixes where the index behind the scales lies)
// xbs: a scale per row and 32-value sub-block (int8 operands only), or null
int32_t plane_gemm_blocks(uint32_t type, int nb, bool gateup, const GemmArgs & k, unsigned blocks, hipStream_t s);
int32_t enqueue_plane_gemm(const tqmoe_bank & b0, const tqmoe_bank * b1, const int8_t * xq, const float * xs, const int * counts, const int * offsets,
                           const int * perm, int experts, int64_t assignments, void * out_f16, int gateup, int shared_expert, int shared_lim, hipStream_t s,
                           const float * xbs) {
    const int nb = gateup || b0.rows % 64 == 0 ? 2 : 1;
    const int units = gateup ? b0.rows / 32 : b0.rows / (32 * nb);
    const int64_t tiles = grouped_row_tiles(assignments, experts);
    // units per item: about sixteen super-block steps of products behind one item's start-up, in a divisor of the units
    int unit_group = std::max(1, std::min(4, 16 / std::max(1, b0.cols / 256)));
    while (units % unit_group) --unit_group;
    GemmArgs k{view(b0), b1 ? view(*b1) : view(b0), xq, xs, counts, offsets, perm, plan_at(xs, tiles * 32, experts), experts, static_cast<uint16_t *>(out_f16),
               units, unit_group, shared_expert, shared_lim, xbs};
    // one block per compute unit (the kernel's registers and LDS allow no second one), walking the work items
    const int cus = cu_count();
    const int64_t most = (tiles / kChunkTiles + experts + 7) / 8 * 8 * (units / unit_group);     // an upper bound of the items
    const unsigned blocks = unsigned(std::min<int64_t>((cus + 7) / 8 * 8, most));
    if (xbs) return plane_gemm_blocks(b0.type, nb, gateup != 0, k, blocks, s);
    switch (b0.type) {
        case TQMOE_IQ4_XS: plane_gemm_launch<WIq4xs>(nb, gateup != 0, k, blocks, s); break;
        case TQMOE_IQ3_S: plane_gemm_launch<WIq3s>(nb, gateup != 0, k, blocks, s); break;
        case TQMOE_Q4_K: plane_gemm_launch<WQ4k>(nb, gateup != 0, k, blocks, s); break;
        case TQMOE_NVFP4G: plane_gemm_launch<WNvfp4>(nb, gateup != 0, k, blocks, s); break;
        case TQMOE_IQ3_XXS: plane_gemm_launch<WIq3xxs>(nb, gateup != 0, k, blocks, s); break;
        case TQMOE_IQ2_XXS: plane_gemm_launch<WIq2xxs>(nb, gateup != 0, k, blocks, s); break;
        case TQMOE_IQ2_XS: plane_gemm_launch<WIq2xs>(nb, gateup != 0, k, blocks, s); break;
        case TQMOE_IQ2_S: plane_gemm_launch<WIq2s>(nb, gateup != 0, k, blocks, s); break;
        case TQMOE_IQ1_S: plane_gemm_launch<WIq1s>(nb, gateup != 0, k, blocks, s); break;
        case TQMOE_IQ4_NL: plane_gemm_launch<WIq4nl>(nb, gateup != 0, k, blocks, s); break;
        default: return -1;
    }
    return 0;
}

}  // namespace tqmoe

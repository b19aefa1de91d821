// Entry helpers of the 8-bit grouped products: the row quantisers, the grouped operand and the per-row-scale products.
#include "prefill_planes_kernels.cuh"

namespace tqmoe {
namespace {

// the largest magnitude over the four lanes that hold a 32-value block (eight values each)
__device__ __forceinline__ float quad_max(float v) {
    v = fmaxf(v, dpp_f<kDppXor1>(v));
    return fmaxf(v, dpp_f<kDppXor2>(v));
}
__device__ __forceinline__ int byte_sum_i8(uint32_t w) { return int(int8_t(w)) + int(int8_t(w >> 8)) + int(int8_t(w >> 16)) + int(int8_t(w >> 24)); }

// rows of 8-bit activations: q = rint(x * 127 / amax) per row, scale = amax / 127 (E4M3: 448 in place of 127); one wave per row.
// BLK: amax and scale per block of 32 values (scale [rows][cols / 32]) and, when asked for, the sums of q over each 16
// values (qsum [rows][cols / 32][2]).
template <int XT, bool F8, bool BLK = false>
__global__ __launch_bounds__(256) void quant_rows_k(const void * __restrict__ x, int64_t rows, int cols, int8_t * __restrict__ q, float * __restrict__ scale,
                                                    int16_t * __restrict__ qsum = nullptr) {
    const int lane = threadIdx.x & 63;
    const int64_t row = int64_t(blockIdx.x) * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int groups = cols / 8;   // 8 consecutive values = natural dwords 2j, 2j + 1 of a 32-block
    if constexpr (BLK) {           // (a block's four lanes enter or leave the loop together: cols is a multiple of 32)
        uint32_t * out = reinterpret_cast<uint32_t *>(q + row * cols);
        for (int gi = lane; gi < groups; gi += 64) {
            float v[8];
            load8<XT>(x, row * cols + gi * 8, v);
            float amax = 0.f;
#pragma unroll
            for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(v[j]));
            amax = quad_max(amax);
            const float mul = amax > 0.f ? 127.f / amax : 0.f;
            const uint32_t w[2] = {pack4_q<false>(v[0] * mul, v[1] * mul, v[2] * mul, v[3] * mul), pack4_q<false>(v[4] * mul, v[5] * mul, v[6] * mul, v[7] * mul)};
            const int blk = gi >> 2, d0 = 2 * (gi & 3);
            out[blk * 8 + plane_pos(d0)] = w[0];
            out[blk * 8 + plane_pos(d0 + 1)] = w[1];
            if ((gi & 3) == 0) scale[row * (cols / 32) + blk] = amax / 127.f;
            if (qsum) {
                int sum = byte_sum_i8(w[0]) + byte_sum_i8(w[1]);
                sum += dpp_i<kDppXor1>(sum);
                if ((gi & 1) == 0) qsum[(row * (cols / 32) + blk) * 2 + ((gi & 3) >> 1)] = int16_t(sum);
            }
        }
        return;
    }
    float amax = 0.f;
    for (int gi = lane; gi < groups; gi += 64) {
        float v[8];
        load8<XT>(x, row * cols + gi * 8, v);
#pragma unroll
        for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(v[j]));
    }
    amax = fmaxf(amax, dpp_f<kDppXor1>(amax));
    amax = fmaxf(amax, dpp_f<kDppXor2>(amax));
    amax = fmaxf(amax, dpp_f<kDppHalfMirror>(amax));
    amax = fmaxf(amax, dpp_f<kDppMirror>(amax));
    amax = fmaxf(amax, __shfl_xor(amax, 16, 64));
    amax = fmaxf(amax, __shfl_xor(amax, 32, 64));
    const float mul = amax > 0.f ? kOperandMax<F8> / amax : 0.f;
    if (lane == 0) scale[row] = amax / kOperandMax<F8>;
    uint32_t * out = reinterpret_cast<uint32_t *>(q + row * cols);
    for (int gi = lane; gi < groups; gi += 64) {
        float v[8];
        load8<XT>(x, row * cols + gi * 8, v);
        const uint32_t w[2] = {pack4_q<F8>(v[0] * mul, v[1] * mul, v[2] * mul, v[3] * mul), pack4_q<F8>(v[4] * mul, v[5] * mul, v[6] * mul, v[7] * mul)};
        const int blk = gi >> 2, d0 = 2 * (gi & 3);
        out[blk * 8 + plane_pos(d0)] = w[0];
        out[blk * 8 + plane_pos(d0 + 1)] = w[1];
    }
}

// inclusive prefix sum over the wave's 64 lanes with DPP moves (rows of 16, then the rows' totals handed on)
template <int N> __device__ __forceinline__ int dpp_row_shr(int v) { return __builtin_amdgcn_update_dpp(0, v, 0x110 + N, 0xF, 0xF, true); }
__device__ __forceinline__ int wave_prefix_sum(int v) {
    v += dpp_row_shr<1>(v);
    v += dpp_row_shr<2>(v);
    v += dpp_row_shr<4>(v);
    v += dpp_row_shr<8>(v);
    v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xA, 0xF, false);   // row_bcast:15 into rows 1 and 3
    v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xC, 0xF, false);   // row_bcast:31 into rows 2 and 3
    return v;
}

__global__ __launch_bounds__(64) void plan_k(const int * __restrict__ counts, int experts, Plan plan) {
    const int lane = threadIdx.x;
    int * tile_base = const_cast<int *>(plan.tile_base), * chunk_base = const_cast<int *>(plan.chunk_base), * chunk_base2 = const_cast<int *>(plan.chunk_base2);
    if (lane < kPlanCounters) plan.counters[lane] = 0;
    int tbase = 0, cbase = 0, cbase2 = 0;
    constexpr int kAhead = 16;   // counts of 16 x 64 experts are loaded in one trip to memory, then scanned 64 at a time
    for (int eb = 0; eb < experts; eb += 64 * kAhead) {
        int cnt[kAhead];
#pragma unroll
        for (int i = 0; i < kAhead; ++i) cnt[i] = counts[min(eb + 64 * i + lane, experts - 1)];
#pragma unroll
        for (int i = 0; i < kAhead; ++i) {
            const int e0 = eb + 64 * i;
            if (e0 >= experts) break;
            const int e = e0 + lane;
            const int tiles = e < experts ? (max(cnt[i], 0) + 31) >> 5 : 0;
            const int chunks = (tiles + kChunkTiles - 1) / kChunkTiles, chunks2 = (tiles + 2 * kChunkTiles - 1) / (2 * kChunkTiles);
            const int ti = wave_prefix_sum(tiles), ci = wave_prefix_sum(chunks), c2 = wave_prefix_sum(chunks2);
            if (e < experts) { tile_base[e] = tbase + ti - tiles; chunk_base[e] = cbase + ci - chunks; chunk_base2[e] = cbase2 + c2 - chunks2; }
            tbase += __builtin_amdgcn_readlane(ti, 63);
            cbase += __builtin_amdgcn_readlane(ci, 63);
            cbase2 += __builtin_amdgcn_readlane(c2, 63);
        }
    }
    if (lane == 0) { tile_base[experts] = tbase; chunk_base[experts] = cbase; chunk_base2[experts] = cbase2; }
}

// Rows of the grouped operand: block b takes rows [8 (b % 4), +8) of row tile b / 4, one wave per two rows. Row i of
// expert e's tiles is assignment perm[offsets[e] + i], its source row a / xdiv. Rows past the expert's count are left as
// they are (their products are never stored).
template <int XT, bool F8, bool BLK = false>
__global__ __launch_bounds__(256) void group_rows_k(const void * __restrict__ x, int cols, const int * __restrict__ counts, const int * __restrict__ offsets,
                                                         const int * __restrict__ perm, int experts, int xdiv, int8_t * __restrict__ q, float * __restrict__ scale,
                                                         Plan plan, float * __restrict__ block_scale = nullptr) {
    const int tile_index = int(blockIdx.x >> 2);
    if (tile_index >= plan.tile_base[experts]) return;
    const int e = owner_of(plan.tile_base, experts, tile_index);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int cnt = counts[e], groups = cols / 8, lt = tile_index - plan.tile_base[e];
    uint32_t * tile = reinterpret_cast<uint32_t *>(q + int64_t(tile_index) * 32 * cols);
#pragma unroll
    for (int rr = 0; rr < 2; ++rr) {
        const int r = int(blockIdx.x & 3) * 8 + wave * 2 + rr;
        const int i = lt * 32 + r;
        if (i >= cnt) break;
        const int64_t row = perm[offsets[e] + i] / xdiv;
        float amax = 0.f;
        if constexpr (!BLK) {
            for (int gi = lane; gi < groups; gi += 64) {
                float v[8];
                load8<XT>(x, row * cols + gi * 8, v);
#pragma unroll
                for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(v[j]));
            }
            amax = wave_max(amax);
        }
        float mul = amax > 0.f ? kOperandMax<F8> / amax : 0.f;
        if (lane == 0) scale[int64_t(tile_index) * 32 + r] = BLK ? 1.f : amax / kOperandMax<F8>;
        for (int gi = lane; gi < groups; gi += 64) {
            float v[8];
            load8<XT>(x, row * cols + gi * 8, v);
            if constexpr (BLK) {   // the block's own scale (its four lanes run together: cols is a multiple of 32)
                amax = 0.f;
#pragma unroll
                for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(v[j]));
                amax = quad_max(amax);
                mul = amax > 0.f ? kOperandMax<F8> / amax : 0.f;
                if ((gi & 3) == 0) block_scale[(int64_t(tile_index) * (cols / 32) + (gi >> 2)) * 32 + r] = amax / kOperandMax<F8>;
            }
            const uint32_t wd[2] = {pack4_q<F8>(v[0] * mul, v[1] * mul, v[2] * mul, v[3] * mul), pack4_q<F8>(v[4] * mul, v[5] * mul, v[6] * mul, v[7] * mul)};
            const int sub = gi >> 2, d0 = 2 * (gi & 3);
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int p = plane_pos(d0 + h);          // dword of the 32-byte block; its half p / 4 is the lane group g
                tile[sub * 256 + ((p >> 2) * 32 + r) * 4 + (p & 3)] = wd[h];
            }
        }
    }
}

// The same for row lengths that are a multiple of 256 up to 2048: one block per row tile. A wave quantises eight rows out of registers
// (one read of the input) into an LDS copy of the tile, every 32-byte block already in operand order; then lane (g, r)
// of every wave moves the 16 bytes of row r, half g of one k-step at a time, so each k-step's 1 KB leaves as one fully
// coalesced store instead of 256 scattered dwords.
template <int XT, int GPL, bool F8, bool BLK = false>   // groups of 8 values per lane: 512 (GPL - 1) < cols <= 512 GPL
__global__ __launch_bounds__(256) void group_rows_tile_k(const void * __restrict__ x, int cols, const int * __restrict__ counts, const int * __restrict__ offsets,
                                                              const int * __restrict__ perm, int experts, int xdiv, int8_t * __restrict__ q, float * __restrict__ scale,
                                                              Plan plan, float * __restrict__ block_scale = nullptr) {
    extern __shared__ __attribute__((aligned(16))) uint8_t tile_rows[];   // [32][cols + 16]
    const int tile_index = int(blockIdx.x);
    if (tile_index >= plan.tile_base[experts]) return;
    const int e = owner_of(plan.tile_base, experts, tile_index);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, stride = cols + 16;
    const int cnt = counts[e], first = (tile_index - plan.tile_base[e]) * 32, off = offsets[e];
    constexpr int kBatch = GPL == 3 ? 2 : 8 / GPL;   // rows whose loads are in flight together: about 64 values per lane
    const int groups = cols / 8;
    for (int r0 = wave * 8; r0 < wave * 8 + 8; r0 += kBatch) {
        if (first + r0 >= cnt) break;
        float v[kBatch][GPL][8];
#pragma unroll
        for (int b = 0; b < kBatch; ++b) {
            const int i = min(first + r0 + b, cnt - 1);          // past the count: a valid row again, not stored
            const int64_t row = perm[off + i] / xdiv;
#pragma unroll
            for (int gq = 0; gq < GPL; ++gq) {
                if (lane + 64 * gq < groups) load8<XT>(x, row * cols + (lane + 64 * gq) * 8, v[b][gq]);
                else
#pragma unroll
                    for (int j = 0; j < 8; ++j) v[b][gq][j] = 0.f;
            }
        }
#pragma unroll
        for (int b = 0; b < kBatch; ++b) {
            const int r = r0 + b;
            float amax = 0.f;
#pragma unroll
            for (int gq = 0; gq < GPL; ++gq)
#pragma unroll
                for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(v[b][gq][j]));
            if constexpr (!BLK) amax = wave_max(amax);
            float mul = amax > 0.f ? kOperandMax<F8> / amax : 0.f;
            // (a scale per block: the four lanes of a block hold its values in the same gq, and take every branch below together)
            float bmax[GPL];
            if constexpr (BLK) {
#pragma unroll
                for (int gq = 0; gq < GPL; ++gq) {
                    float m = 0.f;
#pragma unroll
                    for (int j = 0; j < 8; ++j) m = fmaxf(m, fabsf(v[b][gq][j]));
                    bmax[gq] = quad_max(m);
                }
            }
            if (first + r < cnt) {
                if (lane == 0) scale[int64_t(tile_index) * 32 + r] = BLK ? 1.f : amax / kOperandMax<F8>;
#pragma unroll
                for (int gq = 0; gq < GPL; ++gq) {
                    const int gi = lane + 64 * gq, sub = gi >> 2, d0 = 2 * (gi & 3);
                    if (gi >= groups) break;
                    if constexpr (BLK) {
                        mul = bmax[gq] > 0.f ? kOperandMax<F8> / bmax[gq] : 0.f;
                        if ((gi & 3) == 0) block_scale[(int64_t(tile_index) * (cols / 32) + sub) * 32 + r] = bmax[gq] / kOperandMax<F8>;
                    }
                    const float * vv = v[b][gq];
                    const uint32_t wd[2] = {pack4_q<F8>(vv[0] * mul, vv[1] * mul, vv[2] * mul, vv[3] * mul), pack4_q<F8>(vv[4] * mul, vv[5] * mul, vv[6] * mul, vv[7] * mul)};
#pragma unroll
                    for (int h = 0; h < 2; ++h) *reinterpret_cast<uint32_t *>(tile_rows + r * stride + sub * 32 + plane_pos(d0 + h) * 4) = wd[h];
                }
            }
        }
    }
    __syncthreads();
    const int r = lane & 31, g = lane >> 5;
    if (first + r >= cnt) return;                     // rows past the expert's count are left as they are
    uint4 * dst = reinterpret_cast<uint4 *>(q + int64_t(tile_index) * 32 * cols) + lane;
    const int S = cols / 32;
    for (int ks = wave; ks < S; ks += 4) dst[ks * 64] = *reinterpret_cast<const uint4 *>(tile_rows + r * stride + ks * 32 + g * 16);
}

// The same grouped operand from rows that are already int8 (quant_rows_k's output: one scale per row, the bytes of every
// 32-block in operand order): a pure copy. One block per row tile; lane (g, r) of every wave moves the 16 bytes of row r,
// half g of one k-step at a time, so each k-step's 1 KB is written by one fully coalesced store. When several
// assignments read one input row (xdiv > 1) the row is quantised once instead of once per assignment.
// block_scale: rs holds a scale per row and 32-value block ([rows][cols / 32]); they go to block_scale
// [row tile][block][32 rows] and the rows' own scales are 1.
__global__ __launch_bounds__(256) void gather_rows_i8_k(const int8_t * __restrict__ rq, const float * __restrict__ rs, int cols, const int * __restrict__ counts,
                                                          const int * __restrict__ offsets, const int * __restrict__ perm, int experts, int xdiv,
                                                          int8_t * __restrict__ q, float * __restrict__ scale, Plan plan, float * __restrict__ block_scale = nullptr) {
    const int tile_index = int(blockIdx.x);
    if (tile_index >= plan.tile_base[experts]) return;
    const int e = owner_of(plan.tile_base, experts, tile_index);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, r = lane & 31, g = lane >> 5;
    const int i = (tile_index - plan.tile_base[e]) * 32 + r;
    if (i >= counts[e]) return;                       // rows past the expert's count are left as they are
    const int64_t row = perm[offsets[e] + i] / xdiv;
    const int S = cols / 32;
    if (wave == 0 && g == 0) scale[int64_t(tile_index) * 32 + r] = block_scale ? 1.f : rs[row];
    const uint4 * src = reinterpret_cast<const uint4 *>(rq + row * cols) + g;
    uint4 * dst = reinterpret_cast<uint4 *>(q + int64_t(tile_index) * 32 * cols) + lane;
    for (int ks = wave; ks < S; ks += 4) dst[ks * 64] = src[ks * 2];
    if (block_scale && g == 0)
        for (int ks = wave; ks < S; ks += 4) block_scale[(int64_t(tile_index) * S + ks) * 32 + r] = rs[row * S + ks];
}

// The grouped operand from int8 rows in natural order with scales laid out [rows][cols / 32] (what the reference's activation
// quantiser leaves: quant_act_rows_k, src/formats/weight/quant_u4h.inc:790-822): lane (g, r) reads the two 8-byte halves of
// its 16 operand bytes (values 8 g .. 8 g + 7 and 16 + 8 g .. 16 + 8 g + 7 of the block) and interleaves their dwords.
// per_block: every block's own scale goes to block_scale and the rows' scales are 1; else the row's scale is its first entry.
__global__ __launch_bounds__(256) void gather_rows_natural_k(const int8_t * __restrict__ rq, const float * __restrict__ rs, int cols, const int * __restrict__ counts,
                                                             const int * __restrict__ offsets, const int * __restrict__ perm, int experts, int xdiv,
                                                             int8_t * __restrict__ q, float * __restrict__ scale, Plan plan, float * __restrict__ block_scale) {
    const int tile_index = int(blockIdx.x);
    if (tile_index >= plan.tile_base[experts]) return;
    const int e = owner_of(plan.tile_base, experts, tile_index);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, r = lane & 31, g = lane >> 5;
    const int i = (tile_index - plan.tile_base[e]) * 32 + r;
    if (i >= counts[e]) return;                       // rows past the expert's count are left as they are
    const int64_t row = perm[offsets[e] + i] / xdiv;
    const int S = cols / 32;
    if (wave == 0 && g == 0) scale[int64_t(tile_index) * 32 + r] = block_scale ? 1.f : rs[row * S];
    const uint2 * src = reinterpret_cast<const uint2 *>(rq + row * cols) + g;
    uint4 * dst = reinterpret_cast<uint4 *>(q + int64_t(tile_index) * 32 * cols) + lane;
    for (int ks = wave; ks < S; ks += 4) {
        const uint2 lo = src[ks * 4], hi = src[ks * 4 + 2];
        dst[ks * 64] = make_uint4(lo.x, hi.x, lo.y, hi.y);
    }
    if (block_scale && g == 0)
        for (int ks = wave; ks < S; ks += 4) block_scale[(int64_t(tile_index) * S + ks) * 32 + r] = rs[row * S + ks];
}

}  // namespace

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
// plan_from: the scales of another grouping of the same lists (same counts, same experts, same bound of assignments) whose
// index is read in place of building this one's again; the products on these rows must then be given it as well
int32_t enqueue_group_rows_i8(const void * x, uint32_t xtype, int cols, const int * counts, const int * offsets, const int * perm, int experts,
                              int64_t assignments, int xdiv, int8_t * q, float * scale, hipStream_t s, bool f8, float * block_scale, const float * plan_from) {
    const int64_t tiles = grouped_row_tiles(assignments, experts);
    const Plan plan = plan_at(plan_from ? plan_from : scale, tiles * 32, experts);
    if (!plan_from) plan_k<<<1, 64, 0, s>>>(counts, experts, plan);
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

int32_t enqueue_gather_rows_natural(const int8_t * rq, const float * rs, int cols, const int * counts, const int * offsets, const int * perm, int experts,
                                    int64_t assignments, int xdiv, int8_t * q, float * scale, hipStream_t s, float * block_scale) {
    const int64_t tiles = grouped_row_tiles(assignments, experts);
    const Plan plan = plan_at(scale, tiles * 32, experts);
    plan_k<<<1, 64, 0, s>>>(counts, experts, plan);
    gather_rows_natural_k<<<unsigned(tiles), 256, 0, s>>>(rq, rs, cols, counts, offsets, perm, experts, xdiv, q, scale, plan, block_scale);
    return 0;
}

// bank formats with a plane GEMM: int8 operands (IQ4_XS, IQ4_NL, IQ3_S, IQ3_XXS, IQ2_XXS, IQ2_XS, IQ2_S, IQ1_S, Q4_K, Q5_K, Q4_0, Q8_0) or E4M3
// operands (NVFP4G). Q6_K, Q3_K and Q2_K carry a scale per 16 weights, half the depth of the matrix instruction: their
// grouped products go through the fp16 kernels.
bool plane_gemm_has(uint32_t type) {
    return type == TQMOE_IQ4_XS || type == TQMOE_IQ3_S || type == TQMOE_Q4_K || type == TQMOE_NVFP4G || type == TQMOE_IQ3_XXS || type == TQMOE_IQ2_XXS ||
           type == TQMOE_IQ2_XS || type == TQMOE_IQ2_S || type == TQMOE_IQ1_S || type == TQMOE_IQ4_NL || type == TQMOE_Q5_K || type == TQMOE_Q4_0 || type == TQMOE_Q8_0;
}
bool plane_gemm_is_fp8(uint32_t type) { return type == TQMOE_NVFP4G; }

// assignments = total entries of perm (it fixes where the index behind the scales lies)
// xbs: a scale per row and 32-value sub-block (int8 operands only), or null
int32_t plane_gemm_blocks(uint32_t type, int nb, bool gateup, const GemmArgs & k, unsigned blocks, hipStream_t s);
int32_t plane_gemm_legacy(uint32_t type, int nb, bool gateup, bool blk, const GemmArgs & k, unsigned blocks, hipStream_t s);
int32_t enqueue_plane_gemm(const tqmoe_bank & b0, const tqmoe_bank * b1, const int8_t * xq, const float * xs, const int * counts, const int * offsets,
                           const int * perm, int experts, int64_t assignments, void * out_f16, int gateup, int shared_expert, int shared_lim, hipStream_t s,
                           const float * xbs, Glu glu, int out_bf16, const float * plan_from) {
    const int nb = gateup || b0.rows % 64 == 0 ? 2 : 1;
    const int units = gateup ? b0.rows / 32 : b0.rows / (32 * nb);
    const int64_t tiles = grouped_row_tiles(assignments, experts);
    // units per item: about sixteen super-block steps of products behind one item's start-up, in a divisor of the units
    int unit_group = std::max(1, std::min(4, 16 / std::max(1, b0.cols / 256)));
    while (units % unit_group) --unit_group;
    GemmArgs k{view(b0), b1 ? view(*b1) : view(b0), xq, xs, counts, offsets, perm, plan_at(plan_from ? plan_from : xs, tiles * 32, experts), experts, static_cast<uint16_t *>(out_f16),
               units, unit_group, shared_expert, shared_lim, xbs, glu, out_bf16};
    // one block per compute unit (the kernel's registers and LDS allow no second one), walking the work items
    const int cus = cu_count();
    const int64_t most = (tiles / kChunkTiles + experts + 7) / 8 * 8 * (units / unit_group);     // an upper bound of the items
    const unsigned blocks = unsigned(std::min<int64_t>((cus + 7) / 8 * 8, most));
    if (b0.type == TQMOE_Q5_K || b0.type == TQMOE_Q4_0 || b0.type == TQMOE_Q8_0) return plane_gemm_legacy(b0.type, nb, gateup != 0, xbs != nullptr, k, blocks, s);
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

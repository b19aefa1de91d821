// Prefill-sized expert products of IQ4_XS banks: a grouped int8 x int8 -> int32 GEMM on the matrix pipe.
//
// Operands. Activations are int8 per input row (one fp32 scale per row, amax / 127). The rows of every expert's
// assignments are gathered into tiles of 32 rows, experts in order, each expert padded to whole tiles, and stored
// operand-major: the 1 KB that the 64 lanes of a wave feed to one v_mfma_i32_32x32x32_i8 as operand A (lane = 32 g + r
// holds, for row r and 32-weight sub-block j, the 16 values {8g..8g+7} and {16+8g..16+8g+7} in the byte order of the
// bank's code bytes) is contiguous, sub-blocks in order. A wave then loads its operand with one fully coalesced
// instruction and no shuffle.
// Weights stay exact. An IQ4_XS value is d * (ls - 32) * kv[q]: the product (ls - 32) * kv[q] (13 bits) is split as
// 64 * h + l with h, l int8, taken per sub-block from a 64-entry table of 16-value lookup tables in LDS and applied with
// v_perm_b32. The two planes go through two MFMAs that accumulate over the whole 256-weight super-block, so the scales
// cost no vector instruction per product; per super-block the results fold as acc += d * (64 * acc_h + acc_l) in fp32.
//
// Blocks. A work item is one expert, a chunk of up to kChunkTiles row tiles of its assignments and one unit of weight
// rows: 32 rows of both banks (gate / up, SwiGLU fused) or 64 rows of one bank (down). Resident blocks of eight waves
// take items from counters (one per XCD, so that a chunk's rows stay in one L2). Per super-block the waves decode the
// unit's weights once into a double-buffered LDS stage that every wave then reads as operand B (decoding super-block
// i + 1 overlaps the products of super-block i, one barrier per super-block); a wave multiplies one row tile with the
// weights of both operand slots, so a loaded piece of operand A (prefetched into registers a few k-steps ahead) serves
// four products and SwiGLU pairs values the same lane holds. A chunk of a single row tile has nothing to share: every
// wave then takes the tile against 32 weight rows of its own (four units per item), decoding straight into registers
// with no barrier in the loop.
#include "act_image.cuh"
#include "decode_api.cuh"
#include "formats.cuh"

#include <algorithm>
#include <type_traits>

namespace tqmoe {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kChunkTiles = 8;                // row tiles (of 32 assignments) per chunk
constexpr int kPlanExperts = 1024;              // experts whose index a block keeps in LDS

__device__ __forceinline__ v4i decode16(uint2 c) {
    v4i w;
    uint32_t lo, hi;
    lookup16<kIq4T0, kIq4T1, kIq4T2, kIq4T3>(c.x, lo, hi);
    w[0] = int(lo); w[1] = int(hi);
    lookup16<kIq4T0, kIq4T1, kIq4T2, kIq4T3>(c.y, lo, hi);
    w[2] = int(lo); w[3] = int(hi);
    return w;
}

// rows of int8 activations: q = rint(x * 127 / amax) per row, scale = amax / 127; one wave per row
template <int XT>
__global__ __launch_bounds__(256) void quant_rows_i8_k(const void * __restrict__ x, int64_t rows, int cols, int8_t * __restrict__ q, float * __restrict__ scale) {
    const int lane = threadIdx.x & 63;
    const int64_t row = int64_t(blockIdx.x) * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int groups = cols / 8;   // 8 consecutive values = natural dwords 2j, 2j + 1 of a 32-block
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
    const float mul = amax > 0.f ? 127.f / amax : 0.f;
    if (lane == 0) scale[row] = amax / 127.f;
    uint32_t * out = reinterpret_cast<uint32_t *>(q + row * cols);
    for (int gi = lane; gi < groups; gi += 64) {
        float v[8];
        load8<XT>(x, row * cols + gi * 8, v);
        uint32_t w[2] = {0, 0};
#pragma unroll
        for (int j = 0; j < 8; ++j) w[j >> 2] |= uint32_t(__float2int_rn(v[j] * mul) & 0xFF) << (8 * (j & 3));
        const int blk = gi >> 2, d0 = 2 * (gi & 3);
        out[blk * 8 + plane_pos(d0)] = w[0];
        out[blk * 8 + plane_pos(d0 + 1)] = w[1];
    }
}

// Index of the grouped rows, kept behind the row scales: tile_base[e] = row tiles of the experts before e
// (tiles_e = ceil(count_e / 32)), chunk_base[e] = chunks of kChunkTiles row tiles before e, both with a total at [experts].
// Behind them 16 counters the product kernel hands work out with (zero between launches).
constexpr int kPlanCounters = 16;
struct Plan { const int * tile_base, * chunk_base; int * counters; };
__host__ __device__ inline Plan plan_at(const float * scale, int64_t grouped_rows, int experts) {
    const int * p = reinterpret_cast<const int *>(scale + grouped_rows);
    return Plan{p, p + experts + 1, const_cast<int *>(p) + 2 * (experts + 1)};
}

__global__ __launch_bounds__(64) void plan_k(const int * __restrict__ counts, int experts, int * __restrict__ tile_base, int * __restrict__ chunk_base,
                                             int * __restrict__ counters) {
    const int lane = threadIdx.x;
    if (lane < kPlanCounters) counters[lane] = 0;
    int tbase = 0, cbase = 0;
    for (int e0 = 0; e0 < experts; e0 += 64) {
        const int e = e0 + lane;
        const int tiles = e < experts ? (max(counts[e], 0) + 31) >> 5 : 0;
        const int chunks = (tiles + kChunkTiles - 1) / kChunkTiles;
        int ti = tiles, ci = chunks;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const int a = __shfl_up(ti, d, 64), b = __shfl_up(ci, d, 64);
            if (lane >= d) { ti += a; ci += b; }
        }
        if (e < experts) { tile_base[e] = tbase + ti - tiles; chunk_base[e] = cbase + ci - chunks; }
        tbase += __shfl(ti, 63, 64);
        cbase += __shfl(ci, 63, 64);
    }
    if (lane == 0) { tile_base[experts] = tbase; chunk_base[experts] = cbase; }
}

// largest e in [0, experts) with base[e] <= unit, for unit < base[experts] (experts with no unit share their successor's
// base and are skipped by taking the last of equal entries)
__device__ __forceinline__ int owner_of(const int * __restrict__ base, int experts, int unit) {
    int lo = 0, hi = experts;            // base[lo] <= unit < base[hi]
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (base[mid] <= unit) lo = mid; else hi = mid;
    }
    return lo;
}

// Rows of the grouped operand: block b takes rows [8 (b % 4), +8) of row tile b / 4, one wave per two rows. Row i of
// expert e's tiles is assignment perm[offsets[e] + i], its source row a / xdiv. Rows past the expert's count are left as
// they are (their products are never stored).
template <int XT>
__global__ __launch_bounds__(256) void group_rows_i8_k(const void * __restrict__ x, int cols, const int * __restrict__ counts, const int * __restrict__ offsets,
                                                         const int * __restrict__ perm, int experts, int xdiv, int8_t * __restrict__ q, float * __restrict__ scale,
                                                         Plan plan) {
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
        for (int gi = lane; gi < groups; gi += 64) {
            float v[8];
            load8<XT>(x, row * cols + gi * 8, v);
#pragma unroll
            for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(v[j]));
        }
        amax = wave_max(amax);
        const float mul = amax > 0.f ? 127.f / amax : 0.f;
        if (lane == 0) scale[int64_t(tile_index) * 32 + r] = amax / 127.f;
        for (int gi = lane; gi < groups; gi += 64) {
            float v[8];
            load8<XT>(x, row * cols + gi * 8, v);
            uint32_t wd[2] = {0, 0};
#pragma unroll
            for (int j = 0; j < 8; ++j) wd[j >> 2] |= uint32_t(__float2int_rn(v[j] * mul) & 0xFF) << (8 * (j & 3));
            const int sub = gi >> 2, d0 = 2 * (gi & 3);
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int p = plane_pos(d0 + h);          // dword of the 32-byte block; its half p / 4 is the lane group g
                tile[sub * 256 + ((p >> 2) * 32 + r) * 4 + (p & 3)] = wd[h];
            }
        }
    }
}

// The same for row lengths of 512, 1024 or 2048: one block per row tile. A wave quantises eight rows out of registers
// (one read of the input) into an LDS copy of the tile, every 32-byte block already in operand order; then lane (g, r)
// of every wave moves the 16 bytes of row r, half g of one k-step at a time, so each k-step's 1 KB leaves as one fully
// coalesced store instead of 256 scattered dwords.
template <int XT, int GPL>   // groups of 8 values per lane: cols = 512 GPL
__global__ __launch_bounds__(256) void group_rows_i8_tile_k(const void * __restrict__ x, int cols, const int * __restrict__ counts, const int * __restrict__ offsets,
                                                              const int * __restrict__ perm, int experts, int xdiv, int8_t * __restrict__ q, float * __restrict__ scale,
                                                              Plan plan) {
    extern __shared__ __attribute__((aligned(16))) uint8_t tile_rows[];   // [32][cols + 16]
    const int tile_index = int(blockIdx.x);
    if (tile_index >= plan.tile_base[experts]) return;
    const int e = owner_of(plan.tile_base, experts, tile_index);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, stride = cols + 16;
    const int cnt = counts[e], first = (tile_index - plan.tile_base[e]) * 32, off = offsets[e];
    constexpr int kBatch = 8 / GPL;   // rows whose loads are in flight together: 64 values per lane
    for (int r0 = wave * 8; r0 < wave * 8 + 8; r0 += kBatch) {
        if (first + r0 >= cnt) break;
        float v[kBatch][GPL][8];
#pragma unroll
        for (int b = 0; b < kBatch; ++b) {
            const int i = min(first + r0 + b, cnt - 1);          // past the count: a valid row again, not stored
            const int64_t row = perm[off + i] / xdiv;
#pragma unroll
            for (int gq = 0; gq < GPL; ++gq) load8<XT>(x, row * cols + (lane + 64 * gq) * 8, v[b][gq]);
        }
#pragma unroll
        for (int b = 0; b < kBatch; ++b) {
            const int r = r0 + b;
            float amax = 0.f;
#pragma unroll
            for (int gq = 0; gq < GPL; ++gq)
#pragma unroll
                for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(v[b][gq][j]));
            amax = wave_max(amax);
            const float mul = amax > 0.f ? 127.f / amax : 0.f;
            if (first + r < cnt) {
                if (lane == 0) scale[int64_t(tile_index) * 32 + r] = amax / 127.f;
#pragma unroll
                for (int gq = 0; gq < GPL; ++gq) {
                    const int gi = lane + 64 * gq, sub = gi >> 2, d0 = 2 * (gi & 3);
                    uint32_t wd[2] = {0, 0};
#pragma unroll
                    for (int j = 0; j < 8; ++j) wd[j >> 2] |= uint32_t(__float2int_rn(v[b][gq][j] * mul) & 0xFF) << (8 * (j & 3));
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

// The same grouped operand from rows that are already int8 (quant_rows_i8_k's output: one scale per row, the bytes of every
// 32-block in operand order): a pure copy. One block per row tile; lane (g, r) of every wave moves the 16 bytes of row r,
// half g of one k-step at a time, so each k-step's 1 KB is written by one fully coalesced store. When several
// assignments read one input row (xdiv > 1) the row is quantised once instead of once per assignment.
__global__ __launch_bounds__(256) void gather_rows_i8_k(const int8_t * __restrict__ rq, const float * __restrict__ rs, int cols, const int * __restrict__ counts,
                                                          const int * __restrict__ offsets, const int * __restrict__ perm, int experts, int xdiv,
                                                          int8_t * __restrict__ q, float * __restrict__ scale, Plan plan) {
    const int tile_index = int(blockIdx.x);
    if (tile_index >= plan.tile_base[experts]) return;
    const int e = owner_of(plan.tile_base, experts, tile_index);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, r = lane & 31, g = lane >> 5;
    const int i = (tile_index - plan.tile_base[e]) * 32 + r;
    if (i >= counts[e]) return;                       // rows past the expert's count are left as they are
    const int64_t row = perm[offsets[e] + i] / xdiv;
    if (wave == 0 && g == 0) scale[int64_t(tile_index) * 32 + r] = rs[row];
    const uint4 * src = reinterpret_cast<const uint4 *>(rq + row * cols) + g;
    uint4 * dst = reinterpret_cast<uint4 *>(q + int64_t(tile_index) * 32 * cols) + lane;
    const int S = cols / 32;
    for (int ks = wave; ks < S; ks += 4) dst[ks * 64] = src[ks * 2];
}

struct Where { int expert, local, tile_base; };

struct GemmArgs {
    BankView b0, b1;          // gate and up; down: the same bank twice
    const int8_t * xq;        // grouped operand-major row tiles
    const float * xs;         // [row tiles * 32]
    const int * counts;       // [experts]
    const int * offsets;      // [experts + 1]
    const int * perm;         // assignment indices grouped by expert
    Plan plan;
    int experts;
    uint16_t * out;           // fp16 [assignments][rows]: silu(gate) * up, or the plain product
    int gateup;
    int units;                // weight-row units per expert: rows / 32 (gate / up, and down with NB = 1), rows / 64 (down, NB = 2)
    int shared_expert;        // index of the expert whose rows (gate / up) or columns (down) stop at shared_lim, or -1
    int shared_lim;
};

// 16 codes (two dwords) through the two 16-entry tables of their sub-block scale: h and l planes, 16 int8 each
__device__ __forceinline__ void decode_planes(uint2 c, uint4 th, uint4 tl, v4i & h, v4i & l) {
    const uint32_t cw[2] = {c.x, c.y};
#pragma unroll
    for (int w = 0; w < 2; ++w) {
        const uint32_t i_lo = cw[w] & 0x07070707u, i_hi = (cw[w] >> 4) & 0x07070707u;
        const uint32_t s_lo = ((cw[w] >> 1) & 0x04040404u) | 0x03020100u, s_hi = ((cw[w] >> 5) & 0x04040404u) | 0x03020100u;
        h[2 * w] = int(__builtin_amdgcn_perm(__builtin_amdgcn_perm(th.w, th.z, i_lo), __builtin_amdgcn_perm(th.y, th.x, i_lo), s_lo));
        h[2 * w + 1] = int(__builtin_amdgcn_perm(__builtin_amdgcn_perm(th.w, th.z, i_hi), __builtin_amdgcn_perm(th.y, th.x, i_hi), s_hi));
        l[2 * w] = int(__builtin_amdgcn_perm(__builtin_amdgcn_perm(tl.w, tl.z, i_lo), __builtin_amdgcn_perm(tl.y, tl.x, i_lo), s_lo));
        l[2 * w + 1] = int(__builtin_amdgcn_perm(__builtin_amdgcn_perm(tl.w, tl.z, i_hi), __builtin_amdgcn_perm(tl.y, tl.x, i_hi), s_hi));
    }
}

// The two ways through the kernel (a lone row tile, a shared chunk) must give a row the same bits: the fold of a
// super-block and the epilogue are spelled with explicitly rounded operations, and the product that is converted to fp16
// passes through an opaque register, so that no path turns multiply + convert into one mixed-precision instruction
// (one rounding instead of two: different bits at ties).
__device__ __forceinline__ float fold_sb(float acc, int h, int l, float d) { return __fmaf_rn(float((h << 6) + l), d, acc); }
__device__ __forceinline__ uint16_t to_half_bits(float v) {
    asm volatile("" : "+v"(v));
    return __half_as_ushort(__float2half_rn(v));
}
__device__ __forceinline__ uint16_t swiglu_half(float g_acc, float u_acc, float sc) {
    const float gv = __fmul_rn(g_acc, sc), uv = __fmul_rn(u_acc, sc);
    const float den = __fadd_rn(1.f, __expf(-gv));
    return to_half_bits(__fmul_rn(__fdiv_rn(gv, den), uv));
}
__device__ __forceinline__ uint16_t scaled_half(float acc, float sc) { return to_half_bits(__fmul_rn(acc, sc)); }

__device__ const int8_t kIq4Values[16] = {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113};

// dynamic LDS: [2 stages][NB][plane h, l][8 sub-blocks][64 lanes] v4i of decoded weights.
// 4 * NB waves. Decoding: wave = 4 * slot + quarter decodes sub-blocks 2 quarter, 2 quarter + 1 of operand slot `slot`.
// Products: a wave takes 2 / NB row tiles (tile `wave`, and tile wave + 4 when there is one slot) against every slot.
template <int NB>
__global__ __launch_bounds__(256 * NB) void iq4xs_gemm_k(GemmArgs k) {
    constexpr int THREADS = 256 * NB;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    v4i * bs = reinterpret_cast<v4i *>(lds);
    __shared__ __attribute__((aligned(16))) uint8_t s_tab[64 * 32];   // per 6-bit scale: 16 h bytes, 16 l bytes
    __shared__ int s_asg[kChunkTiles * 32];
    __shared__ float s_scale[kChunkTiles * 32];
    // the experts' index (chunk and tile prefix sums, counts, offsets), copied once: every item looks its expert up, and a
    // binary search is a chain of dependent reads
    __shared__ int s_cbase[kPlanExperts + 1], s_tbase[kPlanExperts + 1], s_cnt[kPlanExperts + 1], s_off[kPlanExperts + 1];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, n = lane & 31, g = lane >> 5;
    const int mg = wave & 3, nbw = wave >> 2;     // row group, operand slot
    const bool cached = k.experts <= kPlanExperts;
    if (cached)
        for (int i = tid; i <= k.experts; i += THREADS) {
            s_cbase[i] = k.plan.chunk_base[i];
            s_tbase[i] = k.plan.tile_base[i];
            s_cnt[i] = i < k.experts ? k.counts[i] : 0;
            s_off[i] = k.offsets[i];
        }

    for (int i = tid; i < 64 * 16; i += THREADS) {
        const int v = int(kIq4Values[i & 15]) * ((i >> 4) - 32);
        const int lo = ((v + 32) & 63) - 32, hi = (v - lo) >> 6;
        s_tab[(i >> 4) * 32 + (i & 15)] = uint8_t(hi);
        s_tab[(i >> 4) * 32 + 16 + (i & 15)] = uint8_t(lo);
    }
    // Work items are (chunk of row tiles, unit of weight rows). Items that share operand A (one chunk, all units) have
    // indices that agree modulo 8, and the blocks that the round-robin of blocks over the 8 XCDs puts on one XCD take the
    // items of one residue from a counter of their own: one XCD's L2 serves a chunk's rows, and a block that finishes
    // early takes more items. The next ticket is fetched under the current item's work. The last block to leave
    // clears the counters for the next launch over these rows.
    __syncthreads();
    const int * cbase = cached ? s_cbase : k.plan.chunk_base, * tbase = cached ? s_tbase : k.plan.tile_base;
    const int * cnts = cached ? s_cnt : k.counts, * offs = cached ? s_off : k.offsets;
    const int n_chunks = cbase[k.experts];
    const int items_padded = (n_chunks + 7) / 8 * 8 * k.units;
    const int S = k.b0.cols / 32, NSB = S / 8, rows = k.b0.rows, tiles_w = rows / 32;
    __shared__ int s_ticket;
    int * ctr = k.plan.counters;
    const int xcd = int(blockIdx.x) & 7;
    int ticket = 0;
    if (tid == 0) ticket = atomicAdd(&ctr[xcd], 1);
    for (;;) {
        __syncthreads();          // the previous item's epilogue has read s_asg / s_scale, the exchange space and s_ticket
        if (tid == 0) s_ticket = ticket;
        __syncthreads();
        const int item = 8 * s_ticket + xcd;
        if (item >= items_padded) break;
        if (tid == 0) ticket = atomicAdd(&ctr[xcd], 1);
        const int unit = (item >> 3) % k.units, chunk = item / (8 * k.units) * 8 + (item & 7);
        if (chunk >= n_chunks) continue;
        const int e = owner_of(cbase, k.experts, chunk);
        const int local = chunk - cbase[e], tile_base = tbase[e];
        const bool is_shared = e == k.shared_expert;
        // gate / up rows of the shared expert beyond its size: no products, zeros stored (the rows are quantised whole later)
        const bool dead = k.gateup && is_shared && unit * 32 >= k.shared_lim;
        const int sb_end = dead ? 0 : !k.gateup && is_shared ? k.shared_lim / 256 : NSB;
        const int cnt = cnts[e], tiles_e = (cnt + 31) >> 5;
        const int first_tile = local * kChunkTiles;                         // of this expert
        const int live_tiles = min(kChunkTiles, tiles_e - first_tile);      // of this block
        // A chunk of one row tile has nothing for the waves to share: every wave then takes the tile against 32 weight
        // rows of its own, four units per item, and the chunk's other item numbers are empty.
        const bool lone = live_tiles == 1 && k.units % 4 == 0;
        if (lone && unit >= k.units / 4) continue;
        for (int i = tid; i < kChunkTiles * 32; i += THREADS) {
            const int idx = first_tile * 32 + i;
            const bool ok = i < live_tiles * 32 && idx < cnt;
            s_asg[i] = ok ? k.perm[offs[e] + idx] : -1;
            s_scale[i] = ok ? k.xs[int64_t(tile_base + first_tile) * 32 + i] : 0.f;
        }
        __syncthreads();
        if (lone) {
            // weight tile of this wave: gate / up: tile 4 unit + mg of bank nbw; down: tile (4 unit + mg) NB + nbw
            const int wt = k.gateup ? 4 * unit + mg : (4 * unit + mg) * NB + nbw;
            const BankView & wbank = nbw ? k.b1 : k.b0;
            const bool wdead = k.gateup && is_shared && wt * 32 >= k.shared_lim;
            const int sbe = wdead ? 0 : !k.gateup && is_shared ? k.shared_lim / 256 : NSB;
            const int64_t wtile_g = int64_t(e) * tiles_w + wt;
            const uint8_t * wcodes = wbank.codes + wtile_g * S * 512 + n * 16 + g * 8;
            const uint8_t * waux = wbank.aux + wtile_g * NSB * 256 + n * 8;
            const int8_t * a_ptr = k.xq + int64_t(tile_base + first_tile) * 32 * k.b0.cols + lane * 16;
            struct Stage { uint2 code[8]; uint2 rec; v4i a[8]; };
            auto fetch1 = [&](int sb, Stage & st) {   // a super-block of the wave's weights and of the row tile
                st.rec = *reinterpret_cast<const uint2 *>(waux + int64_t(sb) * 256);
#pragma unroll
                for (int ib = 0; ib < 8; ++ib) {
                    st.code[ib] = *reinterpret_cast<const uint2 *>(wcodes + (int64_t(sb) * 8 + ib) * 512);
                    st.a[ib] = *reinterpret_cast<const v4i *>(a_ptr + (int64_t(sb) * 8 + ib) * 1024);
                }
            };
            float acc_f[16];
#pragma unroll
            for (int i = 0; i < 16; ++i) acc_f[i] = 0.f;
            auto work1 = [&](int sb, Stage & cur, Stage & nxt) {
                fetch1(min(sb + 1, sbe - 1), nxt);   // past the last one the same again, from the cache: no branch, the same loads in flight on every path
                __builtin_amdgcn_sched_barrier(0);
                const float d = half_bits_to_float(iq4xs_d_bits(cur.rec));
                v16i acc_h = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0}, acc_l = acc_h;
#pragma unroll
                for (int ib = 0; ib < 8; ++ib) {
                    const uint4 * tab = reinterpret_cast<const uint4 *>(s_tab + iq4xs_ls(cur.rec, ib) * 32);
                    v4i h, l;
                    decode_planes(cur.code[ib], tab[0], tab[1], h, l);
                    acc_h = __builtin_amdgcn_mfma_i32_32x32x32_i8(cur.a[ib], h, acc_h, 0, 0, 0);
                    acc_l = __builtin_amdgcn_mfma_i32_32x32x32_i8(cur.a[ib], l, acc_l, 0, 0, 0);
                }
#pragma unroll
                for (int i = 0; i < 16; ++i) acc_f[i] = fold_sb(acc_f[i], acc_h[i], acc_l[i], d);
            };
            if (sbe > 0) {
                Stage s0, s1;
                fetch1(0, s0);
                for (int sb = 0; sb < sbe; sb += 2) {
                    work1(sb, s0, s1);
                    if (sb + 1 < sbe) work1(sb + 1, s1, s0);
                }
            }
            float * ex = reinterpret_cast<float *>(lds);
            if (k.gateup && NB == 2) {   // the up waves hand their sums to the gate waves of the same weight tile
                if (nbw == 1) {
#pragma unroll
                    for (int i = 0; i < 16; ++i) ex[(mg * 16 + i) * 64 + lane] = acc_f[i];
                }
                __syncthreads();
            }
            if (!(k.gateup && NB == 2 && nbw == 1)) {
                int asg[16];
                float scl[16];
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const int m = 8 * (i >> 2) + 4 * g + (i & 3);   // result register i of lane half g: row m of the tile, weight row n
                    asg[i] = s_asg[m];
                    scl[i] = s_scale[m];
                }
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    if (asg[i] < 0) continue;
                    uint16_t * o = k.out + int64_t(asg[i]) * rows;
                    if (k.gateup) o[wt * 32 + n] = swiglu_half(acc_f[i], NB == 2 ? ex[(mg * 16 + i) * 64 + lane] : acc_f[i], scl[i]);
                    else o[wt * 32 + n] = scaled_half(acc_f[i], scl[i]);
                }
            }
            continue;
        }
        // Each wave takes 2 / NB row tiles of the chunk (tile `wave`; with one operand slot also tile wave + 4) against
        // the weights of every operand slot: a loaded piece of operand A serves the products with gate and with up (or
        // with both weight tiles of a down unit), and SwiGLU pairs values the same lane holds.
        constexpr int TPW = 2 / NB;
        const int my_tiles = NB == 2 ? (wave < live_tiles ? 1 : 0) : (wave < live_tiles ? 1 : 0) + (wave + 4 < live_tiles ? 1 : 0);
        const int8_t * a_base = k.xq + int64_t(tile_base + first_tile + wave) * 32 * k.b0.cols + lane * 16;
        const int64_t a_tile = int64_t(4) * 32 * k.b0.cols;

        // the weights this wave decodes for everybody: sub-blocks 2 mg and 2 mg + 1 of operand slot nbw
        // (gate / up: the unit's 32 rows of bank nbw; down: row tile NB * unit + nbw)
        const BankView & bank = nbw ? k.b1 : k.b0;
        const int64_t tile_g = int64_t(e) * tiles_w + (k.gateup ? unit : NB * unit + nbw);
        const uint8_t * codes = bank.codes + tile_g * S * 512 + n * 16 + g * 8;   // sub-block s of the tile: + 512 s; lane = (row n, code half g)
        const uint8_t * aux = bank.aux + tile_g * NSB * 256 + n * 8;              // super-block sb of the tile: + 256 sb
        // the scales d of the rows of both slots, for the fold: lane's weight row n, slot b
        const uint8_t * aux_b[NB];
#pragma unroll
        for (int b = 0; b < NB; ++b)
            aux_b[b] = (b ? k.b1 : k.b0).aux + (int64_t(e) * tiles_w + (k.gateup ? unit : NB * unit + b)) * NSB * 256 + n * 8;

        // The super-block loop is instantiated per number of live row tiles of the wave (0..TPW), so that its body is one
        // straight line of code the scheduler can interleave. Every instance passes the same barriers.
        auto body = [&](auto mt_tag) {
            constexpr int MT = decltype(mt_tag)::value;
            constexpr int MTA = MT ? MT : 1;
            v16i acc_h[MTA][NB], acc_l[MTA][NB];
            float acc_f[MTA][NB][16];
#pragma unroll
            for (int t = 0; t < MTA; ++t)
#pragma unroll
                for (int b = 0; b < NB; ++b)
#pragma unroll
                    for (int i = 0; i < 16; ++i) { acc_f[t][b][i] = 0.f; acc_h[t][b][i] = 0; acc_l[t][b][i] = 0; }

            // the codes and the scale record are fetched one super-block before they are decoded, so that their latency is
            // not waited for
            uint2 f_rec = {0, 0}, f_code[2] = {{0, 0}, {0, 0}};
            uint2 d_rec[NB], d_rec_next[NB];
            auto fetch = [&](int sb) {
                f_rec = *reinterpret_cast<const uint2 *>(aux + int64_t(sb) * 256);
#pragma unroll
                for (int j = 0; j < 2; ++j) f_code[j] = *reinterpret_cast<const uint2 *>(codes + (int64_t(sb) * 8 + 2 * mg + j) * 512);
            };
            auto fetch_d = [&](int sb) {
#pragma unroll
                for (int b = 0; b < NB; ++b) d_rec_next[b] = *reinterpret_cast<const uint2 *>(aux_b[b] + int64_t(sb) * 256);
            };
            auto decode_one = [&](int buf, int j) {
                const int ib = 2 * mg + j;
                const uint4 * tab = reinterpret_cast<const uint4 *>(s_tab + iq4xs_ls(f_rec, ib) * 32);
                v4i h, l;
                decode_planes(f_code[j], tab[0], tab[1], h, l);
                bs[(((buf * NB + nbw) * 2 + 0) * 8 + ib) * 64 + lane] = h;
                bs[(((buf * NB + nbw) * 2 + 1) * 8 + ib) * 64 + lane] = l;
            };
            auto decode_into = [&](int buf) { decode_one(buf, 0); decode_one(buf, 1); };
            // operand A, two k-steps (sub-blocks) per slot, fetched kSlots - 1 slots before its products
            constexpr int kSlots = 4;
            v4i a_reg[kSlots][MTA][2];
            auto load_a = [&](int slot, int pair) {
#pragma unroll
                for (int t = 0; t < MT; ++t)
#pragma unroll
                    for (int h = 0; h < 2; ++h) a_reg[slot][t][h] = *reinterpret_cast<const v4i *>(a_base + t * a_tile + (int64_t(pair) * 2 + h) * 1024);
            };

            const int pairs = sb_end * 4;
            if (sb_end > 0) {
                fetch(0);
                fetch_d(0);
#pragma unroll
                for (int q = 0; q < kSlots - 1; ++q) load_a(q, min(q, pairs - 1));
                decode_into(0);
                fetch(min(1, sb_end - 1));
            }
            __syncthreads();
            for (int sb = 0; sb < sb_end; ++sb) {
                const int buf = sb & 1;
#pragma unroll
                for (int b = 0; b < NB; ++b) d_rec[b] = d_rec_next[b];
                // The decode of the next super-block's two sub-blocks is placed between the groups of products, so that its
                // vector work runs while the matrix pipe works through the group just issued. Past the last super-block the
                // fetch repeats it and the decode fills the stage nobody reads: no branches here.
                fetch_d(min(sb + 1, sb_end - 1));
#pragma unroll
                for (int jp = 0; jp < 4; ++jp) {
                    if (jp == 1) { __builtin_amdgcn_sched_barrier(0); decode_one(buf ^ 1, 0); __builtin_amdgcn_sched_barrier(0); }
                    if (jp == 2) { __builtin_amdgcn_sched_barrier(0); decode_one(buf ^ 1, 1); __builtin_amdgcn_sched_barrier(0); }
                    if (jp == 3) { __builtin_amdgcn_sched_barrier(0); fetch(min(sb + 2, sb_end - 1)); __builtin_amdgcn_sched_barrier(0); }
                    load_a((jp + kSlots - 1) % kSlots, min(sb * 4 + jp + kSlots - 1, pairs - 1));
#pragma unroll
                    for (int h = 0; h < 2; ++h) {
                        const int ib = 2 * jp + h;
#pragma unroll
                        for (int b = 0; b < NB; ++b) {
                            const v4i bh = bs[(((buf * NB + b) * 2 + 0) * 8 + ib) * 64 + lane];
                            const v4i bl = bs[(((buf * NB + b) * 2 + 1) * 8 + ib) * 64 + lane];
#pragma unroll
                            for (int t = 0; t < MT; ++t) {
                                const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
                                acc_h[t][b] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a_reg[jp % kSlots][t][h], bh, ib ? acc_h[t][b] : zero, 0, 0, 0);
                                acc_l[t][b] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a_reg[jp % kSlots][t][h], bl, ib ? acc_l[t][b] : zero, 0, 0, 0);
                            }
                        }
                    }
                }
                // |64 acc_h + acc_l| <= 256 * 127 * 127 * 32 < 2^28: exact in int32, then one rounding into fp32
#pragma unroll
                for (int b = 0; b < NB; ++b) {
                    const float d = half_bits_to_float(iq4xs_d_bits(d_rec[b]));
#pragma unroll
                    for (int t = 0; t < MT; ++t)
#pragma unroll
                        for (int i = 0; i < 16; ++i) acc_f[t][b][i] = fold_sb(acc_f[t][b][i], acc_h[t][b][i], acc_l[t][b][i], d);
                }
                __syncthreads();
            }
            // result register i of lane half g is tile row 8 (i / 4) + 4 g + i % 4, weight row n. The rows' assignments and
            // scales are read first, all at once: a read per element inside the store loop would serialise on LDS latency.
#pragma unroll
            for (int t = 0; t < MT; ++t) {
                int asg[16];
                float scl[16];
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const int m = (wave + 4 * t) * 32 + 8 * (i >> 2) + 4 * g + (i & 3);
                    asg[i] = s_asg[m];
                    scl[i] = s_scale[m];
                }
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    if (asg[i] < 0) continue;
                    uint16_t * o = k.out + int64_t(asg[i]) * rows;
                    if (k.gateup) {
                        o[unit * 32 + n] = swiglu_half(acc_f[t][0][i], acc_f[t][NB - 1][i], scl[i]);
                    } else {
#pragma unroll
                        for (int b = 0; b < NB; ++b) o[(NB * unit + b) * 32 + n] = scaled_half(acc_f[t][b][i], scl[i]);
                    }
                }
            }
        };
        if constexpr (NB == 2) {
            if (my_tiles) body(std::integral_constant<int, 1>{}); else body(std::integral_constant<int, 0>{});
        } else {
            switch (my_tiles) {
                case 0: body(std::integral_constant<int, 0>{}); break;
                case 1: body(std::integral_constant<int, 1>{}); break;
                default: body(std::integral_constant<int, 2>{}); break;
            }
        }
    }   // items
    if (tid == 0) {
        __threadfence();
        if (atomicAdd(&ctr[8], 1) == int(gridDim.x) - 1)
            for (int i = 0; i < kPlanCounters; ++i) atomicExch(&ctr[i], 0);
    }
}

}  // namespace


// ---------------------------------------------------------------------------------------------- entry helpers
int64_t grouped_row_tiles(int64_t assignments, int experts) { return (assignments + 31) / 32 + experts; }

int32_t enqueue_quant_rows_i8(const void * x, uint32_t xtype, int64_t rows, int cols, int8_t * q, float * scale, hipStream_t s) {
    const unsigned blocks = unsigned((rows + 3) / 4);
    switch (xtype) {
        case TQMOE_F32: quant_rows_i8_k<TQMOE_F32><<<blocks, 256, 0, s>>>(x, rows, cols, q, scale); break;
        case TQMOE_F16: quant_rows_i8_k<TQMOE_F16><<<blocks, 256, 0, s>>>(x, rows, cols, q, scale); break;
        default: quant_rows_i8_k<TQMOE_BF16><<<blocks, 256, 0, s>>>(x, rows, cols, q, scale); break;
    }
    return 0;
}

int64_t grouped_scale_words(int64_t assignments, int experts) { return grouped_row_tiles(assignments, experts) * 32 + 2 * (int64_t(experts) + 1) + kPlanCounters; }

int32_t enqueue_group_rows_i8(const void * x, uint32_t xtype, int cols, const int * counts, const int * offsets, const int * perm, int experts,
                              int64_t assignments, int xdiv, int8_t * q, float * scale, hipStream_t s) {
    const int64_t tiles = grouped_row_tiles(assignments, experts);
    const Plan plan = plan_at(scale, tiles * 32, experts);
    plan_k<<<1, 64, 0, s>>>(counts, experts, const_cast<int *>(plan.tile_base), const_cast<int *>(plan.chunk_base), plan.counters);
    if (cols == 512 || cols == 1024 || cols == 2048) {
        const size_t lds = size_t(32) * size_t(cols + 16);
        auto launch = [&](auto kernel) {
            if (lds > 65536) allow_dynamic_lds(reinterpret_cast<const void *>(kernel), 32 * (2048 + 16));
            kernel<<<unsigned(tiles), 256, lds, s>>>(x, cols, counts, offsets, perm, experts, xdiv, q, scale, plan);
        };
#define TQMOE_GROUP_TILE(XT) (cols == 512 ? launch(group_rows_i8_tile_k<XT, 1>) : cols == 1024 ? launch(group_rows_i8_tile_k<XT, 2>) : launch(group_rows_i8_tile_k<XT, 4>))
        switch (xtype) {
            case TQMOE_F32: TQMOE_GROUP_TILE(TQMOE_F32); break;
            case TQMOE_F16: TQMOE_GROUP_TILE(TQMOE_F16); break;
            default: TQMOE_GROUP_TILE(TQMOE_BF16); break;
        }
#undef TQMOE_GROUP_TILE
        return 0;
    }
    const unsigned blocks = unsigned(tiles * 4);
    switch (xtype) {
        case TQMOE_F32: group_rows_i8_k<TQMOE_F32><<<blocks, 256, 0, s>>>(x, cols, counts, offsets, perm, experts, xdiv, q, scale, plan); break;
        case TQMOE_F16: group_rows_i8_k<TQMOE_F16><<<blocks, 256, 0, s>>>(x, cols, counts, offsets, perm, experts, xdiv, q, scale, plan); break;
        default: group_rows_i8_k<TQMOE_BF16><<<blocks, 256, 0, s>>>(x, cols, counts, offsets, perm, experts, xdiv, q, scale, plan); break;
    }
    return 0;
}

int32_t enqueue_gather_rows_i8(const int8_t * rq, const float * rs, int cols, const int * counts, const int * offsets, const int * perm, int experts,
                               int64_t assignments, int xdiv, int8_t * q, float * scale, hipStream_t s) {
    const int64_t tiles = grouped_row_tiles(assignments, experts);
    const Plan plan = plan_at(scale, tiles * 32, experts);
    plan_k<<<1, 64, 0, s>>>(counts, experts, const_cast<int *>(plan.tile_base), const_cast<int *>(plan.chunk_base), plan.counters);
    gather_rows_i8_k<<<unsigned(tiles), 256, 0, s>>>(rq, rs, cols, counts, offsets, perm, experts, xdiv, q, scale, plan);
    return 0;
}

// assignments = total entries of perm (it fixes where the index behind the scales lies)
int32_t enqueue_iq4xs_gemm(const tqmoe_bank & b0, const tqmoe_bank * b1, const int8_t * xq, const float * xs, const int * counts, const int * offsets,
                           const int * perm, int experts, int64_t assignments, void * out_f16, int gateup, int shared_expert, int shared_lim, hipStream_t s) {
    const int nb = gateup || b0.rows % 64 == 0 ? 2 : 1;
    const int units = gateup ? b0.rows / 32 : b0.rows / (32 * nb);
    const int64_t tiles = grouped_row_tiles(assignments, experts);
    GemmArgs k{view(b0), b1 ? view(*b1) : view(b0), xq, xs, counts, offsets, perm, plan_at(xs, tiles * 32, experts), experts, static_cast<uint16_t *>(out_f16),
               gateup, units, shared_expert, shared_lim};
    // one block per compute unit (the kernel's registers and LDS allow no second one), walking the work items
    const int cus = cu_count();
    const int64_t most = (tiles / kChunkTiles + experts + 7) / 8 * 8 * units;     // an upper bound of the items
    const unsigned blocks = unsigned(std::min<int64_t>((cus + 7) / 8 * 8, most));
    const size_t lds = size_t(2) * nb * 2 * 8 * 64 * sizeof(v4i);
    if (nb == 2) {
        allow_dynamic_lds(reinterpret_cast<const void *>(&iq4xs_gemm_k<2>), 65536);
        iq4xs_gemm_k<2><<<blocks, 512, lds, s>>>(k);
    } else {
        iq4xs_gemm_k<1><<<blocks, 256, lds, s>>>(k);
    }
    return 0;
}

}  // namespace tqmoe

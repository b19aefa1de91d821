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
// Blocks. A block takes one expert, a chunk of up to kChunkTiles row tiles of its assignments (kMT per wave) and one
// unit of weight rows: 32 rows of both banks (gate / up, SwiGLU fused) or 64 rows of one bank (down). Per super-block
// the four waves decode the unit's weights once into a double-buffered LDS stage (two k-steps of both operands each)
// that every wave then reads as operand B; decoding super-block i + 1 overlaps the products of super-block i, one barrier
// per super-block. Operand A is prefetched into registers two k-steps ahead.
#include "act_image.cuh"
#include "decode_api.cuh"
#include "formats.cuh"

#include <algorithm>
#include <type_traits>

namespace tqmoe {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kMT = 2;                       // row tiles (of 32 assignments) per wave
constexpr int kGemmWaves = 4;
constexpr int kChunkTiles = kMT * kGemmWaves;   // row tiles per block

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
struct Plan { const int * tile_base, * chunk_base; };
__host__ __device__ inline Plan plan_at(const float * scale, int64_t grouped_rows, int experts) {
    const int * p = reinterpret_cast<const int *>(scale + grouped_rows);
    return Plan{p, p + experts + 1};
}

__global__ __launch_bounds__(64) void plan_k(const int * __restrict__ counts, int experts, int * __restrict__ tile_base, int * __restrict__ chunk_base) {
    const int lane = threadIdx.x;
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

__device__ const int8_t kIq4Values[16] = {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113};

// dynamic LDS: [2 stages][NB][plane h, l][8 sub-blocks][64 lanes] v4i of decoded weights.
// 4 * NB waves: wave = 4 * slot + row group; a wave multiplies its kMT row tiles with the weights of its operand slot
// (gate or up; for down the two row tiles of the unit), so that two waves share a SIMD and one's vector work and loads
// overlap the other's products.
template <int NB>
__global__ __launch_bounds__(256 * NB) void iq4xs_gemm_k(GemmArgs k) {
    constexpr int THREADS = 256 * NB;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    v4i * bs = reinterpret_cast<v4i *>(lds);
    __shared__ __attribute__((aligned(16))) uint8_t s_tab[64 * 32];   // per 6-bit scale: 16 h bytes, 16 l bytes
    __shared__ int s_asg[kChunkTiles * 32];
    __shared__ float s_scale[kChunkTiles * 32];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, n = lane & 31, g = lane >> 5;
    const int mg = wave & 3, nbw = wave >> 2;     // row group, operand slot

    for (int i = tid; i < 64 * 16; i += THREADS) {
        const int v = int(kIq4Values[i & 15]) * ((i >> 4) - 32);
        const int lo = ((v + 32) & 63) - 32, hi = (v - lo) >> 6;
        s_tab[(i >> 4) * 32 + (i & 15)] = uint8_t(hi);
        s_tab[(i >> 4) * 32 + 16 + (i & 15)] = uint8_t(lo);
    }
    // Work items are (chunk of row tiles, unit of weight rows); the blocks of the grid walk them with the grid as stride.
    // Items that share operand A (one chunk, all units) have indices that agree modulo 8, so that with the round-robin of
    // blocks over the 8 XCDs (grid a multiple of 8) one XCD's L2 serves them.
    const int n_chunks = k.plan.chunk_base[k.experts];
    const int items_padded = (n_chunks + 7) / 8 * 8 * k.units;
    const int S = k.b0.cols / 32, NSB = S / 8, rows = k.b0.rows, tiles_w = rows / 32;
    for (int item = int(blockIdx.x); item < items_padded; item += int(gridDim.x)) {
        const int unit = (item >> 3) % k.units, chunk = item / (8 * k.units) * 8 + (item & 7);
        if (chunk >= n_chunks) continue;
        const int e = owner_of(k.plan.chunk_base, k.experts, chunk);
        const int local = chunk - k.plan.chunk_base[e], tile_base = k.plan.tile_base[e];
        __syncthreads();          // the previous item's epilogue has read s_asg / s_scale and the exchange space
        const bool is_shared = e == k.shared_expert;
        // gate / up rows of the shared expert beyond its size: no products, zeros stored (the rows are quantised whole later)
        const bool dead = k.gateup && is_shared && unit * 32 >= k.shared_lim;
        const int sb_end = dead ? 0 : !k.gateup && is_shared ? k.shared_lim / 256 : NSB;
        const int cnt = k.counts[e], tiles_e = (cnt + 31) >> 5;
        const int first_tile = local * kChunkTiles;                         // of this expert
        const int live_tiles = min(kChunkTiles, tiles_e - first_tile);      // of this block
        for (int i = tid; i < kChunkTiles * 32; i += THREADS) {
            const int idx = first_tile * 32 + i;
            const bool ok = i < live_tiles * 32 && idx < cnt;
            s_asg[i] = ok ? k.perm[k.offsets[e] + idx] : -1;
            s_scale[i] = ok ? k.xs[int64_t(tile_base + first_tile) * 32 + i] : 0.f;
        }
        __syncthreads();

        // row tiles mg and mg + 4 of the chunk: a short chunk spreads over the row groups
        const int my_tiles = (mg < live_tiles ? 1 : 0) + (mg + 4 < live_tiles ? 1 : 0);
        static_assert(kMT == 2 && kChunkTiles == 8, "row tile t of a wave is tile mg + 4 t of the chunk");
        const int8_t * a_base = k.xq + int64_t(tile_base + first_tile + mg) * 32 * k.b0.cols + lane * 16;
        const int64_t a_tile = int64_t(4) * 32 * k.b0.cols;

        // weight rows of this wave's operand slot: gate / up: the unit's 32 rows of bank nbw; down: row tile NB * unit + nbw
        const BankView & bank = nbw ? k.b1 : k.b0;
        const int64_t tile_g = int64_t(e) * tiles_w + (k.gateup ? unit : NB * unit + nbw);
        const uint8_t * codes = bank.codes + tile_g * S * 512 + n * 16 + g * 8;   // sub-block s of the tile: + 512 s; lane = (row n, code half g)
        const uint8_t * aux = bank.aux + tile_g * NSB * 256 + n * 8;              // super-block sb of the tile: + 256 sb

        // The super-block loop is instantiated per number of live row tiles of the wave (0..kMT), so that its body is one
        // straight line of code the scheduler can interleave. Every instance passes the same barriers.
        auto body = [&](auto mt_tag) {
            constexpr int MT = decltype(mt_tag)::value;
            constexpr int MTA = MT ? MT : 1;
            v16i acc_h[MTA], acc_l[MTA];
            float acc_f[MTA][16];
#pragma unroll
            for (int t = 0; t < MTA; ++t)
#pragma unroll
                for (int i = 0; i < 16; ++i) { acc_f[t][i] = 0.f; acc_h[t][i] = 0; acc_l[t][i] = 0; }

            // this wave decodes sub-blocks 2 mg and 2 mg + 1 of every super-block of its slot: the codes and the scale
            // record are fetched one super-block before they are decoded, so that their latency is not waited for
            float d_next = 0.f, d_cur = 0.f;
            uint2 f_rec = {0, 0}, f_code[2] = {{0, 0}, {0, 0}};
            auto fetch = [&](int sb) {
                f_rec = *reinterpret_cast<const uint2 *>(aux + int64_t(sb) * 256);
#pragma unroll
                for (int j = 0; j < 2; ++j) f_code[j] = *reinterpret_cast<const uint2 *>(codes + (int64_t(sb) * 8 + 2 * mg + j) * 512);
            };
            auto decode_into = [&](int buf) {
                d_next = half_bits_to_float(iq4xs_d_bits(f_rec));
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    const int ib = 2 * mg + j;
                    const uint4 * tab = reinterpret_cast<const uint4 *>(s_tab + iq4xs_ls(f_rec, ib) * 32);
                    v4i h, l;
                    decode_planes(f_code[j], tab[0], tab[1], h, l);
                    bs[(((buf * NB + nbw) * 2 + 0) * 8 + ib) * 64 + lane] = h;
                    bs[(((buf * NB + nbw) * 2 + 1) * 8 + ib) * 64 + lane] = l;
                }
            };
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
#pragma unroll
                for (int q = 0; q < kSlots - 1; ++q) load_a(q, min(q, pairs - 1));
                decode_into(0);
                fetch(min(1, sb_end - 1));
            }
            __syncthreads();
            for (int sb = 0; sb < sb_end; ++sb) {
                const int buf = sb & 1;
                d_cur = d_next;
                // past the last super-block the fetch repeats it and the decode fills the stage nobody reads: no branches here
                decode_into(buf ^ 1);
                fetch(min(sb + 2, sb_end - 1));
#pragma unroll
                for (int jp = 0; jp < 4; ++jp) {
                    load_a((jp + kSlots - 1) % kSlots, min(sb * 4 + jp + kSlots - 1, pairs - 1));
#pragma unroll
                    for (int h = 0; h < 2; ++h) {
                        const int ib = 2 * jp + h;
                        const v4i bh = bs[(((buf * NB + nbw) * 2 + 0) * 8 + ib) * 64 + lane];
                        const v4i bl = bs[(((buf * NB + nbw) * 2 + 1) * 8 + ib) * 64 + lane];
#pragma unroll
                        for (int t = 0; t < MT; ++t) {
                            const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
                            acc_h[t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a_reg[jp % kSlots][t][h], bh, ib ? acc_h[t] : zero, 0, 0, 0);
                            acc_l[t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a_reg[jp % kSlots][t][h], bl, ib ? acc_l[t] : zero, 0, 0, 0);
                        }
                    }
                }
                // |64 acc_h + acc_l| <= 256 * 127 * 127 * 32 < 2^28: exact in int32, then one rounding into fp32
#pragma unroll
                for (int t = 0; t < MT; ++t)
#pragma unroll
                    for (int i = 0; i < 16; ++i) acc_f[t][i] += float((acc_h[t][i] << 6) + acc_l[t][i]) * d_cur;
                __syncthreads();
            }
            // result register i of lane half g is tile row 8 (i / 4) + 4 g + i % 4, weight row n.
            // gate / up: the up waves hand their sums to the gate waves of the same rows through the (now idle) weight stage.
            float * ex = reinterpret_cast<float *>(lds);
            if (k.gateup && NB == 2) {
                if (nbw == 1) {
#pragma unroll
                    for (int t = 0; t < MT; ++t)
#pragma unroll
                        for (int i = 0; i < 16; ++i) ex[((mg * kMT + t) * 16 + i) * 64 + lane] = acc_f[t][i];
                }
                __syncthreads();
                if (nbw == 1) return;
            }
#pragma unroll
            for (int t = 0; t < MT; ++t) {
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const int m = (mg + 4 * t) * 32 + 8 * (i >> 2) + 4 * g + (i & 3);
                    const int a = s_asg[m];
                    if (a < 0) continue;
                    const float sc = s_scale[m];
                    uint16_t * o = k.out + int64_t(a) * rows;
                    if (k.gateup) {
                        const float gv = acc_f[t][i] * sc, uv = (NB == 2 ? ex[((mg * kMT + t) * 16 + i) * 64 + lane] : acc_f[t][i]) * sc;
                        o[unit * 32 + n] = __half_as_ushort(__float2half_rn(gv / (1.f + expf(-gv)) * uv));
                    } else {
                        o[(NB * unit + nbw) * 32 + n] = __half_as_ushort(__float2half_rn(acc_f[t][i] * sc));
                    }
                }
            }
        };
        static_assert(kMT == 2, "the dispatch below lists the instances");
        switch (my_tiles) {
            case 0: body(std::integral_constant<int, 0>{}); break;
            case 1: body(std::integral_constant<int, 1>{}); break;
            default: body(std::integral_constant<int, 2>{}); break;
        }
    }   // items
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

int64_t grouped_scale_words(int64_t assignments, int experts) { return grouped_row_tiles(assignments, experts) * 32 + 2 * (int64_t(experts) + 1); }

int32_t enqueue_group_rows_i8(const void * x, uint32_t xtype, int cols, const int * counts, const int * offsets, const int * perm, int experts,
                              int64_t assignments, int xdiv, int8_t * q, float * scale, hipStream_t s) {
    const int64_t tiles = grouped_row_tiles(assignments, experts);
    const Plan plan = plan_at(scale, tiles * 32, experts);
    plan_k<<<1, 64, 0, s>>>(counts, experts, const_cast<int *>(plan.tile_base), const_cast<int *>(plan.chunk_base));
    const unsigned blocks = unsigned(tiles * 4);
    switch (xtype) {
        case TQMOE_F32: group_rows_i8_k<TQMOE_F32><<<blocks, 256, 0, s>>>(x, cols, counts, offsets, perm, experts, xdiv, q, scale, plan); break;
        case TQMOE_F16: group_rows_i8_k<TQMOE_F16><<<blocks, 256, 0, s>>>(x, cols, counts, offsets, perm, experts, xdiv, q, scale, plan); break;
        default: group_rows_i8_k<TQMOE_BF16><<<blocks, 256, 0, s>>>(x, cols, counts, offsets, perm, experts, xdiv, q, scale, plan); break;
    }
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
    static const int cus = [] {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        return n;
    }();
    const int64_t most = (tiles / kChunkTiles + experts + 7) / 8 * 8 * units;     // an upper bound of the items
    const unsigned blocks = unsigned(std::min<int64_t>((cus + 7) / 8 * 8, most));
    const size_t lds = size_t(2) * nb * 2 * 8 * 64 * sizeof(v4i);
    if (nb == 2) {
        static const hipError_t once = hipFuncSetAttribute(reinterpret_cast<const void *>(&iq4xs_gemm_k<2>), hipFuncAttributeMaxDynamicSharedMemorySize, 65536);
        (void)once;
        iq4xs_gemm_k<2><<<blocks, 512, lds, s>>>(k);
    } else {
        iq4xs_gemm_k<1><<<blocks, 256, lds, s>>>(k);
    }
    return 0;
}

}  // namespace tqmoe

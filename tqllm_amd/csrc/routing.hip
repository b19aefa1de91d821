// Router logits, softmax + top-k, and the stable token-to-expert dispatch.
#include <atomic>
#include <mutex>

#include "act_image.cuh"
#include "common.cuh"

namespace tqmoe {
namespace {

// ----------------------------------------------------------------------------------------------------- router
// One wave per router row, TOK tokens per pass; each lane owns 8-element chunks lane, lane + 64, ... of the row.
// Sums in fp32; the order (chunks ascending per lane, then a butterfly over lanes) differs from a column-order host
// sum by ordinary fp32 rounding only.
constexpr int kRouterTok = 4;       // tokens per pass of a wave: the router row is read once for them
constexpr int kRouterTokFew = 1;    // decode-sized batches: a wave per (row, token), the latency of a wave's chain is what counts
constexpr int kRouterFew = 7;       // batches up to here take kRouterTokFew
template <int WT, int XT, int TOK>
__global__ __launch_bounds__(256) void router_k(const void * __restrict__ w, const void * __restrict__ shared,
                                                const void * __restrict__ x, float * __restrict__ logits, int h, int e, int n) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int row = blockIdx.x * 4 + wave;  // 0..e (e = the shared gate)
    const int t0 = blockIdx.y * TOK;
    if (row > e) return;                     // whole waves leave together: reductions below see full waves
    const bool has_row = row < e || shared != nullptr;
    const void * wr = row < e ? w : shared;
    const int64_t wbase = row < e ? int64_t(row) * h : 0;
    float acc[TOK];
#pragma unroll
    for (int i = 0; i < TOK; ++i) acc[i] = 0.f;
    if (has_row) {
        // four 512-column steps of loads at a time (one trip to memory for them instead of four), the sums in column order
        // as before; then what is left of the row step by step
        int c = lane * 8;
        if constexpr (TOK > 1) {   // two steps of loads at a time for the four tokens of a pass
            for (; c + 512 < h; c += 2 * 512) {
                float wv[2][8], xv[TOK][2][8];
#pragma unroll
                for (int q = 0; q < 2; ++q) {
                    load8<WT>(wr, wbase + c + 512 * q, wv[q]);
#pragma unroll
                    for (int i = 0; i < TOK; ++i) load8<XT>(x, int64_t(min(t0 + i, n - 1)) * h + c + 512 * q, xv[i][q]);
                }
#pragma unroll
                for (int i = 0; i < TOK; ++i)
#pragma unroll
                    for (int q = 0; q < 2; ++q)
#pragma unroll
                        for (int j = 0; j < 8; ++j) acc[i] = fmaf(wv[q][j], xv[i][q][j], acc[i]);
            }
        }
        if constexpr (TOK == 1) {
            for (; c + 3 * 512 < h; c += 4 * 512) {
                float wv[4][8], xv[4][8];
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    load8<WT>(wr, wbase + c + 512 * q, wv[q]);
                    load8<XT>(x, int64_t(t0) * h + c + 512 * q, xv[q]);
                }
#pragma unroll
                for (int q = 0; q < 4; ++q)
#pragma unroll
                    for (int j = 0; j < 8; ++j) acc[0] = fmaf(wv[q][j], xv[q][j], acc[0]);
            }
        }
        for (; c < h; c += 512) {
            float wv[8];
            load8<WT>(wr, wbase + c, wv);
#pragma unroll
            for (int i = 0; i < TOK; ++i) {
                if (t0 + i < n) {
                    float xv[8];
                    load8<XT>(x, int64_t(t0 + i) * h + c, xv);
#pragma unroll
                    for (int j = 0; j < 8; ++j) acc[i] = fmaf(wv[j], xv[j], acc[i]);
                }
            }
        }
    }
#pragma unroll
    for (int i = 0; i < TOK; ++i) {
        const float s = group_sum<64>(acc[i]);
        if (lane == 0 && t0 + i < n) logits[int64_t(t0 + i) * (e + 1) + row] = s;
    }
}

template <int WT> int32_t launch_router_x(uint32_t xtype, const void * w, const void * sg, const void * x, float * logits,
                                          int h, int e, int n, hipStream_t s) {
    const bool wide = n <= kRouterFew;   // the wide grid of one-token passes
    const int tok = wide ? kRouterTokFew : kRouterTok;
    const dim3 grid(unsigned((e + 1 + 3) / 4), unsigned((n + tok - 1) / tok));
    switch (xtype) {
        case TQMOE_F32:
            if (wide) router_k<WT, TQMOE_F32, kRouterTokFew><<<grid, 256, 0, s>>>(w, sg, x, logits, h, e, n);
            else router_k<WT, TQMOE_F32, kRouterTok><<<grid, 256, 0, s>>>(w, sg, x, logits, h, e, n);
            return 0;
        case TQMOE_F16:
            if (wide) router_k<WT, TQMOE_F16, kRouterTokFew><<<grid, 256, 0, s>>>(w, sg, x, logits, h, e, n);
            else router_k<WT, TQMOE_F16, kRouterTok><<<grid, 256, 0, s>>>(w, sg, x, logits, h, e, n);
            return 0;
        case TQMOE_BF16:
            if (wide) router_k<WT, TQMOE_BF16, kRouterTokFew><<<grid, 256, 0, s>>>(w, sg, x, logits, h, e, n);
            else router_k<WT, TQMOE_BF16, kRouterTok><<<grid, 256, 0, s>>>(w, sg, x, logits, h, e, n);
            return 0;
    }
    return -1;
}

// Router logits of many tokens, bf16 rows on both sides or fp32 rows on both sides: a GEMM on the matrix pipe. bf16 x bf16
// products are exact in fp32, the fp32 instruction multiplies and adds in fp32, and both accumulate in fp32, so the result
// differs from the scalar kernel's only by the order of the sum. A block of four waves takes 64 tokens x 64 router rows, every wave a 32 x 32 quadrant. The kernel is a
// chain of stages (load from memory, store to LDS, multiply), and a stage costs a trip to memory however little it
// multiplies: so a stage is 512 bytes of every row (256 bf16 columns: eight stages at hidden 2048; 128 fp32 columns), the next stage's loads are in registers while
// this one is multiplied, and two blocks fit a compute unit. The shared expert's gate row rides along as a 65th row of the
// last row block (one more matrix instruction per step for two of its waves), so that 512 experts are eight row blocks and
// not nine.
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));
constexpr int kRouterGemmMin = 120000;   // tokens x router rows from which a bf16 router and input take the GEMM (the wave-per-row kernel
                                         // takes 10 us up to 16,000 and grows with tokens x rows)
constexpr int kRgTok = 64, kRgRows = 64, kRgK = 256, kRgPad = kRgK + 8;   // halves per staged row: 16-byte reads of consecutive rows spread over the banks

// F32: the rows are fp32 (h counts 2-byte units here: twice the columns); else bf16.
// KS = 2: eight waves, the second four take the second half of every stage's steps and hand their sums to the first four
// through LDS at the end (first half + second half, a fixed order): for grids that leave most compute units without a
// block, where a block's own chain of stages is the whole time.
template <bool F32, int KS = 1>
__global__ __launch_bounds__(256 * KS) void router_gemm_k(const uint16_t * __restrict__ w, const uint16_t * __restrict__ shared, const uint16_t * __restrict__ x,
                                                       float * __restrict__ logits, int h, int e, int n) {
    __shared__ __attribute__((aligned(16))) uint16_t As[kRgTok][kRgPad];
    __shared__ __attribute__((aligned(16))) uint16_t Bs[kRgRows + 1][kRgPad];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, r = lane & 31, g = lane >> 5;
    const int t0 = int(blockIdx.x) * kRgTok, r0 = int(blockIdx.y) * kRgRows;
    const bool last = blockIdx.y == gridDim.y - 1;     // this block also has row e (the shared gate, or zeros)
    const int mq = wave & 1, nq = (wave >> 1) & 1;     // quadrant: tokens 32 mq.., router rows 32 nq..
    const int kh = wave >> 2;                          // which part of every stage's steps (0 when KS == 1)
    const bool extra = last && nq == 0;
    // staging: thread -> 16-byte piece sp of rows sr, sr + 8 KS, ... of both tiles (a wave's loads cover two whole rows of 512 bytes)
    constexpr int SR = 8 / KS;                         // rows of each tile a thread stages
    const int sp = tid & 31, sr = tid >> 5;
    const uint16_t * a_src[SR], * b_src[SR];
    bool b_zero[SR];
#pragma unroll
    for (int i = 0; i < SR; ++i) {
        a_src[i] = x + int64_t(min(t0 + sr + 8 * KS * i, n - 1)) * h + 8 * sp;   // rows past the end repeat a valid row (not stored)
        const int row = r0 + sr + 8 * KS * i;
        b_zero[i] = row >= e;
        b_src[i] = w + int64_t(min(row, e - 1)) * h + 8 * sp;
    }
    uint4 a_st[SR], b_st[SR], x_st = make_uint4(0, 0, 0, 0);
    auto fetch = [&](int k0) {
        const bool in = k0 + 8 * sp < h;   // the last stage may be narrower
#pragma unroll
        for (int i = 0; i < SR; ++i) {
            a_st[i] = in ? *reinterpret_cast<const uint4 *>(a_src[i] + k0) : make_uint4(0, 0, 0, 0);
            b_st[i] = in && !b_zero[i] ? *reinterpret_cast<const uint4 *>(b_src[i] + k0) : make_uint4(0, 0, 0, 0);
        }
        if (last && tid < 32) x_st = in && shared ? *reinterpret_cast<const uint4 *>(shared + k0 + 8 * sp) : make_uint4(0, 0, 0, 0);
    };
    auto stage = [&]() {
#pragma unroll
        for (int i = 0; i < SR; ++i) {
            *reinterpret_cast<uint4 *>(&As[sr + 8 * KS * i][8 * sp]) = a_st[i];
            *reinterpret_cast<uint4 *>(&Bs[sr + 8 * KS * i][8 * sp]) = b_st[i];
        }
        if (last && tid < 32) *reinterpret_cast<uint4 *>(&Bs[kRgRows][8 * sp]) = x_st;
    };
    v16f acc, accx, acc1, acc2, acc3;   // the last three: fp32 rows only
#pragma unroll
    for (int q = 0; q < 16; ++q) acc[q] = accx[q] = acc1[q] = acc2[q] = acc3[q] = 0.f;
    fetch(0);
    for (int k0 = 0; k0 < h; k0 += kRgK) {
        __syncthreads();          // the previous stage has been multiplied
        stage();
        __syncthreads();
        if (k0 + kRgK < h) fetch(k0 + kRgK);
        const int steps = min(kRgK, h - k0) / 16;
        auto step = [&](int j) {  // operand of lane (r, g): row r, the 16 bytes at halves 16 j + 8 g
            if constexpr (F32) {  // four fp32 columns a lane: four instructions of two columns each, lane half g's s-th with the other half's s-th
                const float4 a = *reinterpret_cast<const float4 *>(&As[mq * 32 + r][16 * j + 8 * g]);
                const float4 b = *reinterpret_cast<const float4 *>(&Bs[nq * 32 + r][16 * j + 8 * g]);
                // four running sums (joined at the end): a quarter of the terms each, and no instruction waits for the one before it
                acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.x, b.x, acc, 0, 0, 0);
                acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a.y, b.y, acc1, 0, 0, 0);
                acc2 = __builtin_amdgcn_mfma_f32_32x32x2f32(a.z, b.z, acc2, 0, 0, 0);
                acc3 = __builtin_amdgcn_mfma_f32_32x32x2f32(a.w, b.w, acc3, 0, 0, 0);
                if (extra) {
                    const float4 bx = *reinterpret_cast<const float4 *>(&Bs[kRgRows][16 * j + 8 * g]);
                    accx = __builtin_amdgcn_mfma_f32_32x32x2f32(a.x, bx.x, accx, 0, 0, 0);
                    accx = __builtin_amdgcn_mfma_f32_32x32x2f32(a.y, bx.y, accx, 0, 0, 0);
                    accx = __builtin_amdgcn_mfma_f32_32x32x2f32(a.z, bx.z, accx, 0, 0, 0);
                    accx = __builtin_amdgcn_mfma_f32_32x32x2f32(a.w, bx.w, accx, 0, 0, 0);
                }
            } else {
                const v8bf a = *reinterpret_cast<const v8bf *>(&As[mq * 32 + r][16 * j + 8 * g]);
                const v8bf b = *reinterpret_cast<const v8bf *>(&Bs[nq * 32 + r][16 * j + 8 * g]);
                acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc, 0, 0, 0);
                if (extra) {      // every column of this product is row e: lane r = 0 keeps it
                    const v8bf bx = *reinterpret_cast<const v8bf *>(&Bs[kRgRows][16 * j + 8 * g]);
                    accx = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, bx, accx, 0, 0, 0);
                }
            }
        };
        if (steps == kRgK / 16) {
#pragma unroll
            for (int j = 0; j < kRgK / 16 / KS; ++j) step(kh * (kRgK / 16 / KS) + j);
        } else {
            const int per = (steps + KS - 1) / KS;
            for (int j = kh * per; j < min(steps, (kh + 1) * per); ++j) step(j);
        }
    }
    if constexpr (F32) {
#pragma unroll
        for (int q = 0; q < 16; ++q) acc[q] = (acc[q] + acc1[q]) + (acc2[q] + acc3[q]);
    }
    if constexpr (KS == 2) {   // the second part's sums to the first part's waves, through the space of the row tiles
        __syncthreads();       // the last stage has been multiplied
        float * ex = reinterpret_cast<float *>(&As[0][0]);   // [quadrant][17 registers][64 lanes] floats: 17.4 KB of As's 33.8 KB
        static_assert(sizeof(As) >= 4 * 17 * 64 * sizeof(float), "exchange space");
        if (kh == 1) {
#pragma unroll
            for (int q = 0; q < 16; ++q) ex[((wave & 3) * 17 + q) * 64 + lane] = acc[q];
            if (extra) {
#pragma unroll
                for (int q = 0; q < 16; ++q) if (r == 0) ex[((wave & 3) * 17 + 16) * 64 + 16 * g + q] = accx[q];
            }
        }
        __syncthreads();
        if (kh == 1) return;
#pragma unroll
        for (int q = 0; q < 16; ++q) acc[q] += ex[((wave & 3) * 17 + q) * 64 + lane];
        if (extra && r == 0) {
#pragma unroll
            for (int q = 0; q < 16; ++q) accx[q] += ex[((wave & 3) * 17 + 16) * 64 + 16 * g + q];
        }
    }
    // result register q of lane half g: token row 8 (q / 4) + 4 g + q % 4 of the 32-row tile, router row r
    const int row = r0 + nq * 32 + r;
#pragma unroll
    for (int q = 0; q < 16; ++q) {
        const int t = t0 + mq * 32 + 8 * (q >> 2) + 4 * g + (q & 3);
        if (t >= n) continue;
        if (row < e) logits[int64_t(t) * (e + 1) + row] = acc[q];
        if (extra && r == 0) logits[int64_t(t) * (e + 1) + e] = accx[q];
    }
}

// ------------------------------------------------------------------------------------------------------ top-k
// One wave per token. Selection rule of the reference: larger probability first, equal probabilities to the lower
// index. Up to 1024 experts the probabilities stay in registers (lane l owns entries l, l + 64, ...) and every
// reduction is a DPP butterfly ending in a scalar broadcast; larger layers keep them in LDS.
template <int CTRL, int ROWS> __device__ __forceinline__ float dpp_keep_f(float v) {   // lanes outside ROWS get their own value back
    return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(v), __float_as_int(v), CTRL, ROWS, 0xF, false));
}
template <int CTRL, int ROWS> __device__ __forceinline__ int dpp_keep_i(int v) { return __builtin_amdgcn_update_dpp(v, v, CTRL, ROWS, 0xF, false); }
__device__ __forceinline__ float wave_max_all(float v) {   // the wave's maximum, the same in every lane
    v = fmaxf(v, dpp_f<kDppXor1>(v));
    v = fmaxf(v, dpp_f<kDppXor2>(v));
    v = fmaxf(v, dpp_f<kDppHalfMirror>(v));
    v = fmaxf(v, dpp_f<kDppMirror>(v));
    v = fmaxf(v, dpp_keep_f<0x142, 0xA>(v));   // row_bcast:15 into rows 1 and 3
    v = fmaxf(v, dpp_keep_f<0x143, 0xC>(v));   // row_bcast:31 into rows 2 and 3
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}
__device__ __forceinline__ int wave_min_all(int v) {
    v = min(v, dpp_i<kDppXor1>(v));
    v = min(v, dpp_i<kDppXor2>(v));
    v = min(v, dpp_i<kDppHalfMirror>(v));
    v = min(v, dpp_i<kDppMirror>(v));
    v = min(v, dpp_keep_i<0x142, 0xA>(v));
    v = min(v, dpp_keep_i<0x143, 0xC>(v));
    return __builtin_amdgcn_readlane(v, 63);
}
__device__ __forceinline__ int wave_max_all_i(int v) {
    v = max(v, dpp_i<kDppXor1>(v));
    v = max(v, dpp_i<kDppXor2>(v));
    v = max(v, dpp_i<kDppHalfMirror>(v));
    v = max(v, dpp_i<kDppMirror>(v));
    v = max(v, dpp_keep_i<0x142, 0xA>(v));
    v = max(v, dpp_keep_i<0x143, 0xC>(v));
    return __builtin_amdgcn_readlane(v, 63);
}
// Selection keys of the softmax top-k. The reference orders by rounded probability, ties to the lower index
// (src/experts/moe.cpp:73-78); exp and the division by the common sum are monotone, so ordering by logit gives the same
// choice whatever exp() the device has, except where two different logits round to one probability. Entries whose
// probability underflowed to zero are all tied there and go by index: they share one key below every logit's.
// A finite float maps to an integer with the same order (-0 counts as +0); the map is its own inverse.
constexpr int kKeyGone = INT_MIN, kKeyZero = INT_MIN + 1;
__device__ __forceinline__ int order_key(float x) { const int i = __float_as_int(x + 0.f); return i ^ ((i >> 31) & 0x7FFFFFFF); }
__device__ __forceinline__ float key_value(int k) { return __int_as_float(k ^ ((k >> 31) & 0x7FFFFFFF)); }

__device__ __forceinline__ float wave_sum_all(float v) {
    v = row_sum16(v);
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x142, 0xA, 0xF, false));
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x143, 0xC, 0xF, false));
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}

struct TopkOut {
    int * ids; float * weights; float * shared_weights;
    int * ext_ids; int extra;          // optional [n][k + 1] copy of the ids with `extra` in the last slot
    const void * x; uint8_t * image;   // optional: the token's input row is written as an activation image row
    int cols;
    int shared_ungated;                // the shared expert has no gate row: its weight is 1, not sigmoid(0)
};
__device__ __forceinline__ float shared_weight_of(const TopkOut & o, float logit) { return o.shared_ungated ? 1.f : 1.f / (1.f + expf(-logit)); }

__device__ __forceinline__ void topk_finish(const TopkOut & o, const float * x_logits, int token, int lane, int e, int k, float scale, float selected) {
    if (lane == 0) {
        const float total = fmaxf(selected, 6.103515625e-5f);
        for (int s = 0; s < k; ++s) {   // the host divides by the clamped sum, then multiplies by the scale
            float v = o.weights[int64_t(token) * k + s] / total;
            if (scale != 0.f && scale != 1.f) v *= scale;
            o.weights[int64_t(token) * k + s] = v;
        }
        if (o.shared_weights) o.shared_weights[token] = shared_weight_of(o, x_logits[e]);
        if (o.ext_ids) o.ext_ids[int64_t(token) * (k + 1) + k] = o.extra;
    }
}

template <int XT> __device__ __forceinline__ void topk_quantise_row(const TopkOut & o, int token, int lane) {
    quantise_row_wave<XT>(o.x, token, o.cols, o.image + int64_t(token) * (o.cols / 32) * kImageSubBytes, lane);
}

// With an activation image to write the block has a second wave that does nothing else: the row's quantisation runs beside
// the selection instead of after it.
template <int R, int XT>
__device__ __forceinline__ void topk_reg_body(const float * __restrict__ logits, const TopkOut & o, int e, int k, float scale) {
    const int token = blockIdx.x, lane = threadIdx.x & 63;
    const float * x = logits + int64_t(token) * (e + 1);
    if (threadIdx.x >= 64) {
        const int S = o.cols / 32;
        if (S <= 64) {   // one block of 32 values per lane
            float xv[32];
            if (lane < S) load_block32<XT>(o.x, int64_t(token) * o.cols + 32 * lane, xv);
            uint8_t * image_row = o.image + int64_t(token) * S * kImageSubBytes;
            const float amax = wave_max(lane < S ? block_amax(xv) : 0.f);
            if (lane < S) quantise_block(xv, image_row, S, lane, amax);
        } else {
            topk_quantise_row<XT>(o, token, lane);
        }
        return;
    }
    const float shared_logit = o.shared_weights ? x[e] : 0.f;
    int key[R];
    float m = -INFINITY, sum = 0.f;
    {
        float l[R];
#pragma unroll
        for (int r = 0; r < R; ++r) { const int j = lane + 64 * r; l[r] = j < e ? x[j] : -INFINITY; m = fmaxf(m, l[r]); }
        m = wave_max_all(m);
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int j = lane + 64 * r;
            const float ex = j < e ? expf(l[r] - m) : 0.f;
            sum += ex;
            key[r] = j < e ? (ex > 0.f ? order_key(l[r]) : kKeyZero) : kKeyGone;   // entries past the end never win
        }
        sum = wave_sum_all(sum);
    }
    float selected = 0.f, my_w = 0.f;   // lane s keeps selection s
    int my_id = 0;
    if (k <= 64) {
        // Every round is a chain of dependent wave reductions, so the rounds carry only what the next round needs: the
        // winner's key stays in lane s and the probabilities are computed for all selections at once afterwards. Equal
        // keys are rare: one ballot tells whether the winner is alone, and only a tie pays for the index reduction.
        int my_key = kKeyZero;
        for (int s = 0; s < k; ++s) {
            int bk = key[0], bi = lane;
#pragma unroll
            for (int r = 1; r < R; ++r) if (key[r] > bk) { bk = key[r]; bi = lane + 64 * r; }   // strict: the lowest index of equal keys
            const int topkey = wave_max_all_i(bk);
            const unsigned long long tie = __ballot(bk == topkey);
            const int best = __popcll(tie) == 1 ? __builtin_amdgcn_readlane(bi, __builtin_ctzll(tie)) : wave_min_all(bk == topkey ? bi : 0x7FFFFFFF);
            if (lane == s) { my_id = best; my_key = topkey; }
#pragma unroll
            for (int r = 0; r < R; ++r) if (lane + 64 * r == best) key[r] = kKeyGone;
        }
        my_w = my_key == kKeyZero ? 0.f : expf(key_value(my_key) - m) / sum;   // the probability, as every entry's would be computed
        for (int s = 0; s < k; ++s) selected += __int_as_float(__builtin_amdgcn_readlane(__float_as_int(my_w), s));   // slot order, as the host sums them
    } else
    for (int s = 0; s < k; ++s) {
        int bk = key[0], bi = lane;
#pragma unroll
        for (int r = 1; r < R; ++r) if (key[r] > bk) { bk = key[r]; bi = lane + 64 * r; }   // strict: the lowest index of equal keys
        const int topkey = wave_max_all_i(bk);
        const int best = wave_min_all(bk == topkey ? bi : 0x7FFFFFFF);
        const float top = topkey == kKeyZero ? 0.f : expf(key_value(topkey) - m) / sum;   // the probability, as every entry's would be computed
        if (lane == (s & 63)) { my_id = best; my_w = top; }
        if (k > 64 && (s & 63) == 63) {   // more selections than lanes: a full set goes out before the lanes are reused
            o.ids[int64_t(token) * k + s - 63 + lane] = my_id;
            o.weights[int64_t(token) * k + s - 63 + lane] = my_w;   // divided below
            if (o.ext_ids) o.ext_ids[int64_t(token) * (k + 1) + s - 63 + lane] = my_id;
        }
        selected += top;                       // slot order, as the host sums the selected weights
#pragma unroll
        for (int r = 0; r < R; ++r) if (lane + 64 * r == best) key[r] = kKeyGone;
    }
    if (k <= 64) {
        // the host divides by the clamped sum, then multiplies by the scale
        const float total = fmaxf(selected, 6.103515625e-5f);
        if (lane < k) {
            float v = my_w / total;
            if (scale != 0.f && scale != 1.f) v *= scale;
            o.ids[int64_t(token) * k + lane] = my_id;
            o.weights[int64_t(token) * k + lane] = v;
            if (o.ext_ids) o.ext_ids[int64_t(token) * (k + 1) + lane] = my_id;
        }
        if (lane == 0) {
            if (o.shared_weights) o.shared_weights[token] = shared_weight_of(o, shared_logit);
            if (o.ext_ids) o.ext_ids[int64_t(token) * (k + 1) + k] = o.extra;
        }
    } else {
        const int done = k & ~63;             // the last partial set
        if (lane < k - done) {
            o.ids[int64_t(token) * k + done + lane] = my_id;
            o.weights[int64_t(token) * k + done + lane] = my_w;
            if (o.ext_ids) o.ext_ids[int64_t(token) * (k + 1) + done + lane] = my_id;
        }
        __threadfence_block();
        topk_finish(o, x, token, lane, e, k, scale, selected);
    }
}

template <int R, int XT>
__global__ __launch_bounds__(128) void topk_reg_k(const float * __restrict__ logits, TopkOut o, int e, int k, float scale) {
    topk_reg_body<R, XT>(logits, o, e, k, scale);
}
// two routings of the same shape in one launch (blockIdx.y picks): this layer's and a prediction of the next layer's
template <int R>
__global__ __launch_bounds__(64) void topk2_reg_k(const float * __restrict__ logits, TopkOut o, const float * __restrict__ logits2, TopkOut o2, int e, int k,
                                                  float scale) {
    if (blockIdx.y == 0) topk_reg_body<R, TQMOE_F32>(logits, o, e, k, scale);
    else topk_reg_body<R, TQMOE_F32>(logits2, o2, e, k, scale);
}

template <int XT>
__global__ __launch_bounds__(64) void topk_lds_k(const float * __restrict__ logits, TopkOut o, int e, int k, float scale) {
    extern __shared__ int keys[];
    const int token = blockIdx.x, lane = threadIdx.x;
    const float * x = logits + int64_t(token) * (e + 1);
    float m = -INFINITY;
    for (int j = lane; j < e; j += 64) m = fmaxf(m, x[j]);
    m = wave_max_all(m);
    float sum = 0.f;
    for (int j = lane; j < e; j += 64) { const float ex = expf(x[j] - m); keys[j] = ex > 0.f ? order_key(x[j]) : kKeyZero; sum += ex; }
    sum = wave_sum_all(sum);
    float selected = 0.f;
    for (int s = 0; s < k; ++s) {
        int bk = kKeyGone, bi = 0x7FFFFFFF;
        for (int j = lane; j < e; j += 64) if (keys[j] > bk) { bk = keys[j]; bi = j; }
        const int topkey = wave_max_all_i(bk);
        const int best = wave_min_all(bk == topkey ? bi : 0x7FFFFFFF);
        const float top = topkey == kKeyZero ? 0.f : expf(key_value(topkey) - m) / sum;
        if (lane == 0) {
            o.ids[int64_t(token) * k + s] = best;
            o.weights[int64_t(token) * k + s] = top;
            if (o.ext_ids) o.ext_ids[int64_t(token) * (k + 1) + s] = best;
        }
        selected += top;
        if ((best & 63) == lane) keys[best] = kKeyGone;
    }
    topk_finish(o, x, token, lane, e, k, scale, selected);
    if (o.image) topk_quantise_row<XT>(o, token, lane);
}

template <int XT> void launch_topk(const float * logits, const TopkOut & o, int e, int k, int n, float scale, hipStream_t s) {
    if (e <= 64) topk_reg_k<1, XT><<<unsigned(n), o.image ? 128 : 64, 0, s>>>(logits, o, e, k, scale);
    else if (e <= 128) topk_reg_k<2, XT><<<unsigned(n), o.image ? 128 : 64, 0, s>>>(logits, o, e, k, scale);
    else if (e <= 256) topk_reg_k<4, XT><<<unsigned(n), o.image ? 128 : 64, 0, s>>>(logits, o, e, k, scale);
    else if (e <= 512) topk_reg_k<8, XT><<<unsigned(n), o.image ? 128 : 64, 0, s>>>(logits, o, e, k, scale);
    else if (e <= 1024) topk_reg_k<16, XT><<<unsigned(n), o.image ? 128 : 64, 0, s>>>(logits, o, e, k, scale);
    else topk_lds_k<XT><<<unsigned(n), 64, size_t(e) * sizeof(float), s>>>(logits, o, e, k, scale);
}

// The reference's other gating functions (src/experts/moe.cpp:22-113): sigmoid, softmax over the selected logits only,
// sqrt(softplus); a selection bias added for the choice but not for the weights; weights left unnormalised on request.
// One wave per token as above; the values of lane's experts (lane, lane + 64, ...) sit in registers for up to 1024
// experts and in LDS beyond. A taken mask replaces the "below every value" marker of the softmax kernel, since biased
// values and raw logits have no lower bound.
struct Gate { const float * bias; int gating, norm; };

__device__ __forceinline__ float gate_value(int gating, float x) {
    if (gating == TQMOE_GATE_SIGMOID) return 1.0f / (1.0f + expf(-x));
    if (gating == TQMOE_GATE_SQRT_SOFTPLUS) return sqrtf(x > 0.f ? x + log1pf(expf(-x)) : log1pf(expf(x)));
    return x;   // softmax over the selection: the logits themselves
}

// lane 0 finishes a token with more selections than lanes from the raw weights in memory, in slot order as the host does
__device__ void gated_finish_serial(float * w, int k, const Gate & g, float scale) {
    if (g.gating == TQMOE_GATE_SOFTMAX_WEIGHT) {
        float mx = -INFINITY, sum = 0.f;
        for (int s = 0; s < k; ++s) mx = fmaxf(mx, w[s]);
        for (int s = 0; s < k; ++s) { w[s] = expf(w[s] - mx); sum += w[s]; }
        for (int s = 0; s < k; ++s) w[s] = w[s] / sum;
    }
    if (g.norm) {
        float sum = 0.f;
        for (int s = 0; s < k; ++s) sum += w[s];
        sum = fmaxf(sum, 6.103515625e-5f);
        for (int s = 0; s < k; ++s) w[s] = w[s] / sum;
    }
    if (scale != 0.f && scale != 1.f) for (int s = 0; s < k; ++s) w[s] *= scale;
}

// sum over lanes 0 .. k - 1 in lane order (the host's slot order), k <= 64
__device__ __forceinline__ float slot_order_sum(float v, int k) {
    float sum = 0.f;
    for (int s = 0; s < k; ++s) sum += __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), s));
    return sum;
}

template <int R, int XT>   // R = 0: values in LDS, ceil(e / 64) per lane
__global__ __launch_bounds__(64) void topk_gated_k(const float * __restrict__ logits, TopkOut o, Gate g, int e, int k, float scale) {
    extern __shared__ float gated_lds[];
    constexpr bool kLds = R == 0;
    constexpr int kRegs = kLds ? 1 : R;
    const int token = blockIdx.x, lane = threadIdx.x;
    const float * x = logits + int64_t(token) * (e + 1);
    const int per_lane = kLds ? (e + 63) / 64 : R;
    float p_reg[kRegs], v_reg[kRegs];
    float * p_lds = gated_lds + lane, * v_lds = gated_lds + 64 * per_lane + lane;   // entry r of a lane at [64 r]: no bank conflicts
    auto P = [&](int r) -> float & { if constexpr (kLds) return p_lds[64 * r]; else return p_reg[r]; };
    auto V = [&](int r) -> float & { if constexpr (kLds) return v_lds[64 * r]; else return v_reg[r]; };

    const float shared_logit = o.shared_weights ? x[e] : 0.f;
    float m = -INFINITY;
#pragma unroll
    for (int r = 0; r < per_lane; ++r) { const int j = lane + 64 * r; P(r) = j < e ? x[j] : -INFINITY; m = fmaxf(m, P(r)); }
    if (g.gating == TQMOE_GATE_SOFTMAX) {
        m = wave_max_all(m);
        float sum = 0.f;
#pragma unroll
        for (int r = 0; r < per_lane; ++r) { const int j = lane + 64 * r; P(r) = j < e ? expf(P(r) - m) : 0.f; sum += P(r); }
        sum = wave_sum_all(sum);
#pragma unroll
        for (int r = 0; r < per_lane; ++r) P(r) = P(r) / sum;
    } else {
#pragma unroll
        for (int r = 0; r < per_lane; ++r) P(r) = gate_value(g.gating, P(r));
    }
#pragma unroll
    for (int r = 0; r < per_lane; ++r) { const int j = lane + 64 * r; V(r) = g.bias && j < e ? P(r) + g.bias[j] : P(r); }
    uint64_t taken = 0;   // bit r: entry r of this lane is chosen already or lies past the end
#pragma unroll
    for (int r = 0; r < per_lane; ++r) if (lane + 64 * r >= e) taken |= uint64_t(1) << r;

    float selected = 0.f, my_w = 0.f;   // lane s keeps selection s
    int my_id = 0;
    for (int s = 0; s < k; ++s) {
        float bv = -INFINITY;
        int bi = 0x7FFFFFFF;
#pragma unroll
        for (int r = 0; r < per_lane; ++r)   // strict: the lowest index of equal values
            if (!(taken >> r & 1) && (bi == 0x7FFFFFFF || V(r) > bv)) { bv = V(r); bi = lane + 64 * r; }
        const float top = wave_max_all(bv);
        const int best = wave_min_all(bv == top && bi != 0x7FFFFFFF ? bi : 0x7FFFFFFF);
        float wv = 0.f;
#pragma unroll
        for (int r = 0; r < per_lane; ++r) if (lane + 64 * r == best) { wv = P(r); taken |= uint64_t(1) << r; }
        const float w = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(wv), best & 63));   // the unbiased value
        if (lane == (s & 63)) { my_id = best; my_w = w; }
        if (k > 64 && (s & 63) == 63) {   // more selections than lanes: a full set goes out before the lanes are reused
            o.ids[int64_t(token) * k + s - 63 + lane] = my_id;
            o.weights[int64_t(token) * k + s - 63 + lane] = my_w;
            if (o.ext_ids) o.ext_ids[int64_t(token) * (k + 1) + s - 63 + lane] = my_id;
        }
        selected += w;   // slot order, as the host sums the selected weights
    }
    if (k <= 64) {
        if (g.gating == TQMOE_GATE_SOFTMAX_WEIGHT) {
            const float mx = wave_max_all(lane < k ? my_w : -INFINITY);
            my_w = lane < k ? expf(my_w - mx) : 0.f;
            my_w = my_w / slot_order_sum(my_w, k);
            selected = slot_order_sum(my_w, k);
        }
        if (g.norm) my_w = my_w / fmaxf(selected, 6.103515625e-5f);
        if (scale != 0.f && scale != 1.f) my_w *= scale;
        if (lane < k) {
            o.ids[int64_t(token) * k + lane] = my_id;
            o.weights[int64_t(token) * k + lane] = my_w;
            if (o.ext_ids) o.ext_ids[int64_t(token) * (k + 1) + lane] = my_id;
        }
    } else {
        const int done = k & ~63;             // the last partial set
        if (lane < k - done) {
            o.ids[int64_t(token) * k + done + lane] = my_id;
            o.weights[int64_t(token) * k + done + lane] = my_w;
            if (o.ext_ids) o.ext_ids[int64_t(token) * (k + 1) + done + lane] = my_id;
        }
        __threadfence_block();
        if (lane == 0) gated_finish_serial(o.weights + int64_t(token) * k, k, g, scale);
    }
    if (lane == 0) {
        if (o.shared_weights) o.shared_weights[token] = shared_weight_of(o, shared_logit);
        if (o.ext_ids) o.ext_ids[int64_t(token) * (k + 1) + k] = o.extra;
    }
    if (o.image) topk_quantise_row<XT>(o, token, lane);
}

template <int XT> void launch_topk_gated(const float * logits, const TopkOut & o, const Gate & g, int e, int k, int n, float scale, hipStream_t s) {
    if (e <= 64) topk_gated_k<1, XT><<<unsigned(n), 64, 0, s>>>(logits, o, g, e, k, scale);
    else if (e <= 128) topk_gated_k<2, XT><<<unsigned(n), 64, 0, s>>>(logits, o, g, e, k, scale);
    else if (e <= 256) topk_gated_k<4, XT><<<unsigned(n), 64, 0, s>>>(logits, o, g, e, k, scale);
    else if (e <= 512) topk_gated_k<8, XT><<<unsigned(n), 64, 0, s>>>(logits, o, g, e, k, scale);
    else if (e <= 1024) topk_gated_k<16, XT><<<unsigned(n), 64, 0, s>>>(logits, o, g, e, k, scale);
    else topk_gated_k<0, XT><<<unsigned(n), 64, size_t((e + 63) / 64) * 128 * sizeof(float), s>>>(logits, o, g, e, k, scale);
}

// --------------------------------------------------------------------------------------------------- dispatch
// Stable counting sort of the assignments by expert. Chunks of kChunk consecutive assignments; pass 1 counts each
// chunk's experts in LDS, pass 2 turns the per-chunk counts into exclusive prefixes (and counts / offsets), pass 3
// places every assignment at offsets[e] + prefix[chunk][e] + its rank among the chunk's earlier assignments of the
// same expert. Ranks come from ballots (lower lanes of the same expert) and a per-expert running count in LDS that
// waves add to in wave order, so no ordering is left to atomics. A single chunk runs all three passes in one block.
constexpr int kChunk = 1024;

__device__ __forceinline__ void zero_lds(int * a, int n) {
    for (int j = threadIdx.x; j < n; j += blockDim.x) a[j] = 0;
}

// exclusive scan over e of run[0..E) into out[0..E], out[E] = total; one block, E <= 4096, scratch >= blockDim ints
__device__ void block_exclusive_scan(const int * run, int * out, int E, int * scratch) {
    const int tid = threadIdx.x, nt = blockDim.x;
    const int per = (E + nt - 1) / nt, lo = min(tid * per, E), hi = min(lo + per, E);
    int s = 0;
    for (int j = lo; j < hi; ++j) s += run[j];
    scratch[tid] = s;
    __syncthreads();
    for (int d = 1; d < nt; d <<= 1) {  // Hillis-Steele inclusive scan of the per-thread sums
        const int v = tid >= d ? scratch[tid - d] : 0;
        __syncthreads();
        scratch[tid] += v;
        __syncthreads();
    }
    int base = tid ? scratch[tid - 1] : 0;
    for (int j = lo; j < hi; ++j) { out[j] = base; base += run[j]; }
    if (tid == nt - 1) out[E] = scratch[nt - 1];
    __syncthreads();
}

__global__ __launch_bounds__(256) void dispatch_count_k(const int * __restrict__ ids, int * __restrict__ chunk_counts, int A, int E) {
    extern __shared__ int hist[];
    zero_lds(hist, E);
    __syncthreads();
    const int base = blockIdx.x * kChunk;
    for (int i = threadIdx.x; i < kChunk; i += 256) {
        const int a = base + i;
        if (a < A) { const int e = ids[a]; if (e >= 0 && e < E) atomicAdd(&hist[e], 1); }
    }
    __syncthreads();
    for (int j = threadIdx.x; j < E; j += 256) chunk_counts[int64_t(blockIdx.x) * E + j] = hist[j];
}

__global__ __launch_bounds__(1024) void dispatch_scan_k(int * __restrict__ chunk_counts, int * __restrict__ counts,
                                                       int * __restrict__ offsets, int chunks, int E) {
    extern __shared__ int sm[];  // E totals, then 1024 scratch
    for (int e = threadIdx.x; e < E; e += blockDim.x) {
        int run = 0;
        for (int b = 0; b < chunks; ++b) {
            const int v = chunk_counts[int64_t(b) * E + e];
            chunk_counts[int64_t(b) * E + e] = run;
            run += v;
        }
        sm[e] = run;
        counts[e] = run;
    }
    __syncthreads();
    block_exclusive_scan(sm, offsets, E, sm + E);
}

// places one chunk; run[] = per-expert running count inside the chunk (LDS, zeroed by the caller)
__device__ void place_chunk(const int * __restrict__ ids, const int * __restrict__ offsets, const int * __restrict__ prefix,
                            int * __restrict__ perm, int * __restrict__ groups, int capacity, int base, int A, int E, int * run) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
    for (int i0 = 0; i0 < kChunk && base + i0 < A; i0 += blockDim.x) {
        const int a = base + i0 + threadIdx.x;
        int e = a < A ? ids[a] : -1;
        if (e >= E) e = -1;
        // rank of this lane among the wave's earlier lanes of the same expert, and the size of its group
        int rank = 0, size = 0;
        bool last = false;
        unsigned long long todo = __ballot(e >= 0);
        while (todo) {
            const int leader = __ffsll(todo) - 1;
            const int v = __shfl(e, leader, 64);
            const unsigned long long same = __ballot(e == v);
            if (e == v) {
                rank = __popcll(same & ((1ull << lane) - 1ull));
                size = __popcll(same);
                last = (63 - __clzll(same)) == lane;
            }
            todo &= ~same;
        }
        for (int w = 0; w < waves; ++w) {  // waves take their turn in index order
            if (wave == w && e >= 0) {
                const int slot = (prefix ? prefix[e] : 0) + run[e] + rank;
                if (perm) perm[offsets[e] + slot] = a;
                if (groups && slot < capacity) groups[int64_t(e) * capacity + slot] = a;
            }
            __syncthreads();
            if (wave == w && e >= 0 && last) run[e] += size;
            __syncthreads();
        }
    }
}

__global__ __launch_bounds__(256) void dispatch_place_k(const int * __restrict__ ids, const int * __restrict__ offsets,
                                                        const int * __restrict__ chunk_prefix, int * __restrict__ perm,
                                                        int * __restrict__ groups, int capacity, int A, int E) {
    extern __shared__ int run[];
    zero_lds(run, E);
    __syncthreads();
    place_chunk(ids, offsets, chunk_prefix + int64_t(blockIdx.x) * E, perm, groups, capacity, blockIdx.x * kChunk, A, E, run);
}

// Pass 2 and 3 in one launch for up to kWideExperts experts: a block of sixteen waves takes a chunk, one wave per 64
// consecutive assignments. Every block sums the per-chunk counts itself (the chunks before it: where its assignments
// start inside each expert; all chunks: the experts' offsets), the waves rank their assignments with ballots all at
// once and leave their group sizes in a per-wave histogram, and a prefix over the waves in index order gives every
// assignment its place. Nothing is left to the order of atomics.
constexpr int kWideExperts = 1024, kWideWaves = kChunk / 64;

__global__ __launch_bounds__(1024) void dispatch_place_wide_k(const int * __restrict__ ids, const int * __restrict__ chunk_counts, int * __restrict__ counts,
                                                              int * __restrict__ offsets, int * __restrict__ perm, int * __restrict__ groups, int capacity,
                                                              int A, int E, int chunks) {
    extern __shared__ int sm[];   // start E + 1 | total E | scratch 1024 | hist kWideWaves x E
    int * start = sm, * total = sm + E + 1, * scratch = total + E, * hist = scratch + 1024;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, chunk = blockIdx.x;
    for (int j = tid; j < E; j += 1024) {
        int before = 0, all = 0;
        for (int b0 = 0; b0 < chunks; b0 += 16) {   // sixteen loads in flight: the loop is latency, not bandwidth
            int v[16];
#pragma unroll
            for (int q = 0; q < 16; ++q) v[q] = b0 + q < chunks ? chunk_counts[int64_t(b0 + q) * E + j] : 0;
#pragma unroll
            for (int q = 0; q < 16; ++q) { all += v[q]; before += b0 + q < chunk ? v[q] : 0; }
        }
        total[j] = all;
        hist[j] = before;          // parked here until the offsets are known
    }
    for (int j = tid; j < kWideWaves * E; j += 1024) if (j >= E) hist[j] = 0;
    __syncthreads();
    // the assignment's rank among the wave's earlier lanes of the same expert, and the size of its group
    const int a = chunk * kChunk + tid;
    int e = a < A ? ids[a] : -1;
    if (e >= E) e = -1;
    int rank = 0, size = 0;
    bool last = false;
    unsigned long long todo = __ballot(e >= 0);
    while (todo) {
        const int leader = __ffsll(todo) - 1;
        const int v = __shfl(e, leader, 64);
        const unsigned long long same = __ballot(e == v);
        if (e == v) {
            rank = __popcll(same & ((1ull << lane) - 1ull));
            size = __popcll(same);
            last = (63 - __clzll(same)) == lane;
        }
        todo &= ~same;
    }
    const int before_e = e >= 0 ? hist[e] : 0;   // row 0 of hist still holds the chunks before this one
    __syncthreads();
    for (int j = tid; j < E; j += 1024) hist[j] = 0;
    block_exclusive_scan(total, start, E, scratch);   // ends with a barrier
    if (e >= 0 && last) hist[wave * E + e] = size;
    __syncthreads();
    if (e >= 0) {
        int slot = before_e + rank;
        for (int w = 0; w < wave; ++w) slot += hist[w * E + e];
        if (perm) perm[start[e] + slot] = a;
        if (groups && slot < capacity) groups[int64_t(e) * capacity + slot] = a;
    }
    if (chunk == 0) {
        for (int j = tid; j < E; j += 1024) { counts[j] = total[j]; if (offsets) offsets[j] = start[j]; }
        if (tid == 0 && offsets) offsets[E] = start[E];
    }
}

// A <= kChunk: everything in one block
__global__ __launch_bounds__(256) void dispatch_small_k(const int * __restrict__ ids, int * __restrict__ counts, int * __restrict__ offsets,
                                                        int * __restrict__ perm, int * __restrict__ groups, int capacity, int A, int E) {
    extern __shared__ int sm[];  // hist E, offs E + 1, scratch 256
    int * hist = sm, * offs = sm + E, * scratch = sm + 2 * E + 1;
    zero_lds(hist, E);
    __syncthreads();
    for (int a = threadIdx.x; a < A; a += 256) { const int e = ids[a]; if (e >= 0 && e < E) atomicAdd(&hist[e], 1); }
    __syncthreads();
    block_exclusive_scan(hist, offs, E, scratch);
    for (int j = threadIdx.x; j < E; j += 256) { counts[j] = hist[j]; if (offsets) offsets[j] = offs[j]; }
    if (threadIdx.x == 0 && offsets) offsets[E] = offs[E];
    __syncthreads();
    zero_lds(hist, E);
    __syncthreads();
    place_chunk(ids, offs, nullptr, perm, groups, capacity, 0, A, E, hist);
}

}  // namespace
}  // namespace tqmoe

using namespace tqmoe;

extern "C" uint32_t tqmoe_abi_version(void) { return TQMOE_ABI_VERSION; }

extern "C" int32_t tqmoe_router(const void * router, uint32_t wtype, const void * shared_gate, const void * x, uint32_t xtype,
                                float * logits, int32_t hidden, int32_t experts, int32_t n, void * stream, tqmoe_error * err) {
    if (!router || !x || !logits || hidden <= 0 || experts <= 0 || n <= 0) return fail(err, TQMOE_E_ARG, "tqmoe_router: invalid shape or pointer");
    if (hidden % 8) return fail(err, TQMOE_E_ARG, "tqmoe_router: hidden must be a multiple of 8");
    if ((wtype != TQMOE_F32 && wtype != TQMOE_BF16) || !is_act_type(xtype)) return fail(err, TQMOE_E_UNSUPPORTED, "tqmoe_router: unsupported element type");
    if ((n + kRouterTok - 1) / kRouterTok > 65535) return fail(err, TQMOE_E_ARG, "tqmoe_router: too many tokens for one call");
    if (int32_t rc = need_device(err, "tqmoe_router")) return rc;
    const hipStream_t s = static_cast<hipStream_t>(stream);
    if (wtype == xtype && (wtype == TQMOE_BF16 || wtype == TQMOE_F32) && int64_t(n) * (experts + 1) >= kRouterGemmMin && hidden % 64 == 0) {
        const dim3 grid(unsigned((n + kRgTok - 1) / kRgTok), unsigned((experts + kRgRows - 1) / kRgRows));
        const uint16_t * w16 = static_cast<const uint16_t *>(router), * s16 = static_cast<const uint16_t *>(shared_gate), * x16 = static_cast<const uint16_t *>(x);
        // a layer of few experts has few blocks: eight waves a block then, the steps of every stage split between two sets
        // of four (decided by the router rows alone, so that a token's logits do not depend on the batch around it)
        const bool split = grid.y <= 2;
        if (wtype == TQMOE_F32) {
            if (split) router_gemm_k<true, 2><<<grid, 512, 0, s>>>(w16, s16, x16, logits, 2 * hidden, experts, n);
            else router_gemm_k<true><<<grid, 256, 0, s>>>(w16, s16, x16, logits, 2 * hidden, experts, n);
        } else {
            if (split) router_gemm_k<false, 2><<<grid, 512, 0, s>>>(w16, s16, x16, logits, hidden, experts, n);
            else router_gemm_k<false><<<grid, 256, 0, s>>>(w16, s16, x16, logits, hidden, experts, n);
        }
        return launched(err, "tqmoe_router");
    }
    if (wtype == TQMOE_F32) launch_router_x<TQMOE_F32>(xtype, router, shared_gate, x, logits, hidden, experts, n, s);
    else launch_router_x<TQMOE_BF16>(xtype, router, shared_gate, x, logits, hidden, experts, n, s);
    return launched(err, "tqmoe_router");
}

// top-k with the optional extras of the whole-layer path: extended ids and the input rows' activation image
namespace tqmoe {
int32_t enqueue_topk(const float * logits, int32_t * ids, float * weights, float * shared_weights, int32_t * ext_ids, int32_t extra, const void * x,
                     uint32_t xtype, int32_t cols, void * image, int32_t experts, int32_t topk, int32_t n, float scale, int32_t gating,
                     const float * bias, int32_t norm, hipStream_t s, int32_t shared_ungated) {
    const TopkOut o{ids, weights, shared_weights, ext_ids, extra, x, static_cast<uint8_t *>(image), cols, shared_ungated};
    const uint32_t xt = image ? xtype : uint32_t(TQMOE_F32);
    if (gating == TQMOE_GATE_SOFTMAX && !bias && norm) {   // the common case has its own kernel
        switch (xt) {
            case TQMOE_F32: launch_topk<TQMOE_F32>(logits, o, experts, topk, n, scale, s); break;
            case TQMOE_F16: launch_topk<TQMOE_F16>(logits, o, experts, topk, n, scale, s); break;
            default: launch_topk<TQMOE_BF16>(logits, o, experts, topk, n, scale, s); break;
        }
        return 0;
    }
    const Gate g{bias, gating, norm};
    switch (xt) {
        case TQMOE_F32: launch_topk_gated<TQMOE_F32>(logits, o, g, experts, topk, n, scale, s); break;
        case TQMOE_F16: launch_topk_gated<TQMOE_F16>(logits, o, g, experts, topk, n, scale, s); break;
        default: launch_topk_gated<TQMOE_BF16>(logits, o, g, experts, topk, n, scale, s); break;
    }
    return 0;
}
}  // namespace tqmoe

extern "C" int32_t tqmoe_topk(const float * logits, int32_t * ids, float * weights, float * shared_weights, int32_t experts,
                              int32_t topk, int32_t n, float scale, void * stream, tqmoe_error * err) {
    if (!logits || !ids || !weights || experts <= 0 || experts > 4096 || topk <= 0 || topk > experts || n <= 0)
        return fail(err, TQMOE_E_ARG, "tqmoe_topk: invalid shape or pointer");
    if (int32_t rc = need_device(err, "tqmoe_topk")) return rc;
    enqueue_topk(logits, ids, weights, shared_weights, nullptr, 0, nullptr, TQMOE_F32, 0, nullptr, experts, topk, n, scale, TQMOE_GATE_SOFTMAX, nullptr, 1,
                 static_cast<hipStream_t>(stream), 0);
    return launched(err, "tqmoe_topk");
}

// The reference's moe_topk2 (src/experts/moe_kernels.cuh:24-25, src/experts/moe.cu:261-263): moe_topk on two routings in
// one launch, at most 1024 experts.
extern "C" int32_t tqmoe_topk2(const float * logits, int32_t * ids, float * weights, float * shared_weights, const float * logits2, int32_t * ids2,
                               float * weights2, float * shared_weights2, int32_t experts, int32_t topk, int32_t n, float scale, void * stream,
                               tqmoe_error * err) {
    if (!logits || !ids || !weights || !logits2 || !ids2 || !weights2 || experts <= 0 || experts > 1024 || topk <= 0 || topk > experts || n <= 0)
        return fail(err, TQMOE_E_ARG, "tqmoe_topk2: invalid shape or pointer (at most 1024 experts)");
    if (int32_t rc = need_device(err, "tqmoe_topk2")) return rc;
    const TopkOut o{ids, weights, shared_weights, nullptr, 0, nullptr, nullptr, 0, 0}, o2{ids2, weights2, shared_weights2, nullptr, 0, nullptr, nullptr, 0, 0};
    const dim3 grid(unsigned(n), 2);
    const hipStream_t s = static_cast<hipStream_t>(stream);
    if (experts <= 64) topk2_reg_k<1><<<grid, 64, 0, s>>>(logits, o, logits2, o2, experts, topk, scale);
    else if (experts <= 128) topk2_reg_k<2><<<grid, 64, 0, s>>>(logits, o, logits2, o2, experts, topk, scale);
    else if (experts <= 256) topk2_reg_k<4><<<grid, 64, 0, s>>>(logits, o, logits2, o2, experts, topk, scale);
    else if (experts <= 512) topk2_reg_k<8><<<grid, 64, 0, s>>>(logits, o, logits2, o2, experts, topk, scale);
    else topk2_reg_k<16><<<grid, 64, 0, s>>>(logits, o, logits2, o2, experts, topk, scale);
    return launched(err, "tqmoe_topk2");
}

extern "C" int32_t tqmoe_topk_gated(const float * logits, const float * probs_bias, int32_t gating, int32_t norm_weights, int32_t * ids, float * weights,
                                    float * shared_weights, int32_t experts, int32_t topk, int32_t n, float scale, void * stream, tqmoe_error * err) {
    if (!logits || !ids || !weights || experts <= 0 || experts > 4096 || topk <= 0 || topk > experts || n <= 0)
        return fail(err, TQMOE_E_ARG, "tqmoe_topk_gated: invalid shape or pointer");
    if (gating < TQMOE_GATE_SOFTMAX || gating > TQMOE_GATE_SQRT_SOFTPLUS) return fail(err, TQMOE_E_UNSUPPORTED, "tqmoe_topk_gated: unsupported gating function %d", gating);
    if (int32_t rc = need_device(err, "tqmoe_topk_gated")) return rc;
    enqueue_topk(logits, ids, weights, shared_weights, nullptr, 0, nullptr, TQMOE_F32, 0, nullptr, experts, topk, n, scale, gating, probs_bias, norm_weights != 0,
                 static_cast<hipStream_t>(stream), 0);
    return launched(err, "tqmoe_topk_gated");
}

extern "C" size_t tqmoe_dispatch_workspace_bytes(int32_t experts, int32_t n, int32_t topk) {
    if (experts <= 0 || n <= 0 || topk <= 0) return 0;
    const int64_t A = int64_t(n) * topk, chunks = (A + kChunk - 1) / kChunk;
    return chunks <= 1 ? 16 : size_t(chunks) * size_t(experts) * sizeof(int);
}

// Scratch of tqmoe_dispatch_static: the per-chunk counts (and, for a caller that passes no offsets array, the offsets the
// placement of more than 1024 experts reads), in the library's own device image (every GPU the library runs on holds its
// copy until the process ends). In host code the array's name is not a device address: the address on the current device
// comes from hipGetSymbolAddress, once per device, and only that pointer is handed to the kernels.
constexpr int kStaticInts = 1 << 20;                 // 4 MiB: chunks x experts may not exceed it
constexpr int kStaticOffsets = 4352;                 // behind them: room for the offsets of up to 4096 experts
static __device__ __align__(256) int scratch[kStaticInts + kStaticOffsets];

namespace tqmoe {
namespace {
// the launches of tqmoe_dispatch; cc: chunks x experts ints of scratch for more than one chunk. offsets and perm may be
// null where the caller only wants counts and groups (spare_offsets: experts + 1 ints the scan may use instead).
int32_t enqueue_dispatch(const int32_t * ids, int32_t * counts, int32_t * offsets, int32_t * perm, int32_t * groups, int32_t capacity, int32_t experts,
                         int A, int chunks, int * cc, int * spare_offsets, hipStream_t s, tqmoe_error * err, const char * what) {
    if (chunks == 1) {
        dispatch_small_k<<<1, 256, size_t(2 * experts + 1 + 256) * sizeof(int), s>>>(ids, counts, offsets, perm, groups, capacity, A, experts);
        return launched(err, what);
    }
    dispatch_count_k<<<unsigned(chunks), 256, size_t(experts) * sizeof(int), s>>>(ids, cc, A, experts);
    if (experts <= kWideExperts) {
        const size_t lds = size_t(2 * experts + 1 + 1024 + kWideWaves * experts) * sizeof(int);
        allow_dynamic_lds(reinterpret_cast<const void *>(&dispatch_place_wide_k), int((2 * kWideExperts + 1 + 1024 + kWideWaves * kWideExperts) * sizeof(int)));
        dispatch_place_wide_k<<<unsigned(chunks), 1024, lds, s>>>(ids, cc, counts, offsets, perm, groups, capacity, A, experts, chunks);
        return launched(err, what);
    }
    int32_t * offs = offsets ? offsets : spare_offsets;
    dispatch_scan_k<<<1, 1024, size_t(experts + 1024) * sizeof(int), s>>>(cc, counts, offs, chunks, experts);
    dispatch_place_k<<<unsigned(chunks), 256, size_t(experts) * sizeof(int), s>>>(ids, offs, cc, perm, groups, capacity, A, experts);
    return launched(err, what);
}

// Address of ::scratch on each device: looked up once (under the mutex), read without a lock afterwards.
constexpr int kMaxDevices = 64;
std::atomic<int *> g_scratch_ptr[kMaxDevices];
std::mutex g_scratch_mutex;

int32_t static_scratch(int ** out, tqmoe_error * err) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return fail(err, TQMOE_E_DEVICE, "tqmoe_dispatch_static: no usable current device");
    int * p = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!p) {
        std::lock_guard<std::mutex> lock(g_scratch_mutex);
        p = g_scratch_ptr[dev].load(std::memory_order_relaxed);
        if (!p) {
            void * sym = nullptr;
            const hipError_t rc = hipGetSymbolAddress(&sym, HIP_SYMBOL(scratch));
            if (rc != hipSuccess || !sym) return fail(err, TQMOE_E_DEVICE, "tqmoe_dispatch_static: hipGetSymbolAddress: %s", hipGetErrorString(rc));
            p = static_cast<int *>(sym);
            g_scratch_ptr[dev].store(p, std::memory_order_release);
        }
    }
    *out = p;
    return 0;
}

// counts[ids[i]] += 1 as 64-bit counters (a routing profile that runs on over many calls)
__global__ __launch_bounds__(256) void count_k(const int * __restrict__ ids, unsigned long long * __restrict__ counts, int count) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < count) { const int e = ids[i]; if (e >= 0) atomicAdd(counts + e, 1ull); }
}

// The decode grouping maps of one routed call, one block. Assignment a has slot s = slot_of[ids[a]] (-1 for a skipped id).
// The assignments of a slot, in ascending a, are cut into runs of kDedupCols; the run is a group, groups are numbered by
// their first assignment. Every thread walks the slots of the assignments before it (LDS broadcast reads), which gives its
// rank in its slot and the assignment that opened its run; a block-wide prefix over the opening flags numbers the groups.
constexpr int kDedupCols = 8, kDedupStride = 2 + 2 * kDedupCols;
__global__ __launch_bounds__(1024) void dedup_maps_k(const int * __restrict__ ids, const int * __restrict__ slot_of, int count, int topk,
                                                     int * __restrict__ slots, int * __restrict__ gu, int * __restrict__ dn, int groups) {
    __shared__ int s_slot[1024], s_group[1024], s_wave[16];
    const int a = threadIdx.x, lane = a & 63, wave = a >> 6;
    for (int i = a; i < groups * kDedupStride; i += 1024) { if (gu) gu[i] = -1; if (dn) dn[i] = -1; }
    int s = -1;
    if (a < count) { const int e = ids[a]; s = e >= 0 ? slot_of[e] : -1; if (slots) slots[a] = s; }
    s_slot[a] = a < count ? s : -1;
    __syncthreads();
    int rank = 0, total = 0, opener = a;
    if (s >= 0) {
        for (int b = 0; b < count; ++b) {
            if (s_slot[b] != s) continue;
            if (b < a) { if ((rank & (kDedupCols - 1)) == 0) opener = b; ++rank; }
            ++total;
        }
        if ((rank & (kDedupCols - 1)) == 0) opener = a;
    }
    const bool opens = s >= 0 && (rank & (kDedupCols - 1)) == 0;
    const unsigned long long m = __ballot(opens);
    if (lane == 0) s_wave[wave] = __popcll(m);
    __syncthreads();
    int g = __popcll(m & ((1ull << lane) - 1ull));
    for (int w = 0; w < wave; ++w) g += s_wave[w];
    s_group[a] = g;                 // meaningful where the thread opens a group
    __syncthreads();
    if (s < 0) return;
    const int col = rank & (kDedupCols - 1), first = rank - col;
    int * maps[2] = {gu, dn};
#pragma unroll
    for (int part = 0; part < 2; ++part) {
        int * e = maps[part];
        if (!e) continue;
        e += int64_t(s_group[opener]) * kDedupStride;
        if (col == 0) { e[0] = s; e[1] = min(kDedupCols, total - first); }
        e[2 + col] = part ? a : a / topk;
        e[2 + kDedupCols + col] = a;
    }
}
}  // namespace
}  // namespace tqmoe

extern "C" int32_t tqmoe_dispatch(const int32_t * ids, int32_t * counts, int32_t * offsets, int32_t * perm, int32_t * groups,
                                  int32_t capacity, int32_t experts, int32_t n, int32_t topk, void * workspace, size_t workspace_bytes,
                                  void * stream, tqmoe_error * err) {
    if (!ids || !counts || !offsets || !perm || experts <= 0 || experts > 4096 || n <= 0 || topk <= 0 || (groups && capacity <= 0))
        return fail(err, TQMOE_E_ARG, "tqmoe_dispatch: invalid shape or pointer");
    const int64_t A64 = int64_t(n) * topk;
    if (A64 > (1 << 30)) return fail(err, TQMOE_E_ARG, "tqmoe_dispatch: too many assignments");
    const int A = int(A64), chunks = (A + kChunk - 1) / kChunk;
    if (int32_t rc = need_device(err, "tqmoe_dispatch")) return rc;
    const hipStream_t s = static_cast<hipStream_t>(stream);
    if (chunks > 1 && (!workspace || workspace_bytes < tqmoe_dispatch_workspace_bytes(experts, n, topk)))
        return fail(err, TQMOE_E_WORKSPACE, "tqmoe_dispatch: workspace of %zu bytes needed", tqmoe_dispatch_workspace_bytes(experts, n, topk));
    return enqueue_dispatch(ids, counts, offsets, perm, groups, capacity, experts, A, chunks, static_cast<int *>(workspace), nullptr, s, err, "tqmoe_dispatch");
}

extern "C" int32_t tqmoe_dispatch_static(const int32_t * ids, int32_t * counts, int32_t * offsets, int32_t * perm, int32_t * groups,
                                         int32_t capacity, int32_t experts, int32_t n, int32_t topk, void * stream, tqmoe_error * err) {
    if (!ids || !counts || experts <= 0 || experts > 4096 || n <= 0 || topk <= 0 || (groups && capacity <= 0) || (!groups && !perm))
        return fail(err, TQMOE_E_ARG, "tqmoe_dispatch_static: invalid shape or pointer");
    const int64_t A64 = int64_t(n) * topk, chunks64 = (A64 + kChunk - 1) / kChunk;
    if (A64 > (1 << 30)) return fail(err, TQMOE_E_ARG, "tqmoe_dispatch_static: too many assignments");
    if (chunks64 > 1 && chunks64 * experts > kStaticInts)
        return fail(err, TQMOE_E_WORKSPACE, "tqmoe_dispatch_static: %lld assignments x %d experts need %lld scratch ints, the built-in scratch holds %d "
                    "(use tqmoe_dispatch with a workspace)", (long long)A64, experts, (long long)(chunks64 * experts), kStaticInts);
    int * cc = nullptr;
    if (int32_t rc = static_scratch(&cc, err)) return rc;
    return enqueue_dispatch(ids, counts, offsets, perm, groups, capacity, experts, int(A64), int(chunks64), cc, cc + kStaticInts,
                            static_cast<hipStream_t>(stream), err, "tqmoe_dispatch_static");
}

extern "C" int32_t tqmoe_static_scratch_init(tqmoe_error * err) {
    int * p = nullptr;
    if (int32_t rc = need_device(err, "tqmoe_static_scratch_init")) return rc;
    return static_scratch(&p, err) ? TQMOE_E_DEVICE : ok(err);
}

extern "C" int32_t tqmoe_count(const int32_t * ids, uint64_t * counts, int32_t count, void * stream, tqmoe_error * err) {
    if (!ids || !counts || count <= 0) return fail(err, TQMOE_E_ARG, "tqmoe_count: invalid size or pointer");
    if (int32_t rc = need_device(err, "tqmoe_count")) return rc;
    count_k<<<unsigned((count + 255) / 256), 256, 0, static_cast<hipStream_t>(stream)>>>(ids, reinterpret_cast<unsigned long long *>(counts), count);
    return launched(err, "tqmoe_count");
}

extern "C" int32_t tqmoe_dedup_maps(const int32_t * ids, const int32_t * slot_of, int32_t count, int32_t topk, int32_t * slots, int32_t * gu, int32_t * dn,
                                    int32_t groups, void * stream, tqmoe_error * err) {
    if (!ids || !slot_of || count <= 0 || count > 1024 || topk <= 0 || groups < count) return fail(err, TQMOE_E_ARG, "tqmoe_dedup_maps: invalid shape");
    if (int32_t rc = need_device(err, "tqmoe_dedup_maps")) return rc;
    dedup_maps_k<<<1, 1024, 0, static_cast<hipStream_t>(stream)>>>(ids, slot_of, count, topk, slots, gu, dn, groups);
    return launched(err, "tqmoe_dedup_maps");
}

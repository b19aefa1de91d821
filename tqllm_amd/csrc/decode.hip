// Decode-sized expert products: HBM-streaming matrix-vector kernels over the bank layout.
//
// Arithmetic. The input row is held as an "activation image": per 32 values a scale s = amax / 16383 and the integers
// q = rint(x / s) split into two int8 planes, q = 128 * hi + lo with 0 <= lo < 128. A weight sub-block is turned into
// int8 table values in registers (v_perm_b32 lookups for the 4-bit code books, LDS lattice reads for IQ3_S), and the
// product of the two is taken with v_dot4_i32_i8: sum(w * q) = 128 * dot(w, hi) + dot(w, lo), exact in int32. One
// fp32 multiply per sub-block applies weight scale * s. Against an fp32 product the only approximation is the 15-bit
// rounding of x relative to its block maximum (2^-15 relative), three orders below the layer tolerance.
//
// Mapping. A lane owns sub-block(s) sl, sl + LPR, ... of every row it visits, so its slice of the activation image stays
// in registers for the whole kernel and each row costs one 16-byte (12 for IQ3_S) code load per owned sub-block. LPR
// consecutive lanes cover one row; a wave covers 64 / LPR rows per step and finishes each row with a DPP butterfly.
#include "formats.cuh"

namespace tqmoe {
int32_t check_bank(const tqmoe_bank * b, const char * what, tqmoe_error * err);  // bank.hip

namespace {

constexpr int kImageSubBytes = 72;  // 32 B hi plane, 32 B lo plane, fp32 scale, fp32 sum(q) * scale

struct ActBlock { int hi[8], lo[8]; float scale, sum; };

__device__ __forceinline__ void load_act_block(const uint8_t * __restrict__ image_row, int S, int s, ActBlock & b) {
    const uint4 * p = reinterpret_cast<const uint4 *>(image_row + int64_t(s) * 64);
    const uint4 a0 = p[0], a1 = p[1], a2 = p[2], a3 = p[3];
    b.hi[0] = a0.x; b.hi[1] = a0.y; b.hi[2] = a0.z; b.hi[3] = a0.w; b.hi[4] = a1.x; b.hi[5] = a1.y; b.hi[6] = a1.z; b.hi[7] = a1.w;
    b.lo[0] = a2.x; b.lo[1] = a2.y; b.lo[2] = a2.z; b.lo[3] = a2.w; b.lo[4] = a3.x; b.lo[5] = a3.y; b.lo[6] = a3.z; b.lo[7] = a3.w;
    const float2 t = *reinterpret_cast<const float2 *>(image_row + int64_t(S) * 64 + int64_t(s) * 8);
    b.scale = t.x;
    b.sum = t.y;
}
__device__ __forceinline__ void zero_act_block(ActBlock & b) {
#pragma unroll
    for (int i = 0; i < 8; ++i) { b.hi[i] = 0; b.lo[i] = 0; }
    b.scale = 0.f;
    b.sum = 0.f;
}

// 32 values -> image sub-block. v: the values; planes 64 B; trailer 8 B.
__device__ __forceinline__ void quantise_block(const float (&v)[32], uint8_t * planes, uint8_t * trailer) {
    float amax = 0.f;
#pragma unroll
    for (int i = 0; i < 32; ++i) amax = fmaxf(amax, fabsf(v[i]));
    const float scale = amax * (1.f / 16383.f), inv = amax > 0.f ? 16383.f / amax : 0.f;
    uint32_t hi[8], lo[8];
    int qsum = 0;
#pragma unroll
    for (int d = 0; d < 8; ++d) {
        hi[d] = 0;
        lo[d] = 0;
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            const int q = __float2int_rn(v[4 * d + b] * inv);
            qsum += q;
            hi[d] |= uint32_t((q >> 7) & 0xFF) << (8 * b);
            lo[d] |= uint32_t(q & 127) << (8 * b);
        }
    }
    uint4 * p = reinterpret_cast<uint4 *>(planes);
    p[0] = make_uint4(hi[0], hi[1], hi[2], hi[3]);
    p[1] = make_uint4(hi[4], hi[5], hi[6], hi[7]);
    p[2] = make_uint4(lo[0], lo[1], lo[2], lo[3]);
    p[3] = make_uint4(lo[4], lo[5], lo[6], lo[7]);
    *reinterpret_cast<float2 *>(trailer) = make_float2(scale, float(qsum) * scale);
}

template <int XT>
__global__ __launch_bounds__(256) void quant_act_k(const void * __restrict__ x, int n, int cols, uint8_t * __restrict__ image) {
    const int S = cols / 32;
    const int64_t idx = int64_t(blockIdx.x) * 256 + threadIdx.x;
    if (idx >= int64_t(n) * S) return;
    const int64_t row = idx / S;
    const int s = int(idx % S);
    float v[32];
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        float t[8];
        load8<XT>(x, row * cols + 32 * s + 8 * c, t);
#pragma unroll
        for (int j = 0; j < 8; ++j) v[8 * c + j] = t[j];
    }
    uint8_t * base = image + row * int64_t(S) * kImageSubBytes;
    quantise_block(v, base + int64_t(s) * 64, base + int64_t(S) * 64 + int64_t(s) * 8);
}

// ------------------------------------------------------------------------------------------ sub-block products
// dot of one weight sub-block (row `row` of the stacked matrix, sub-block s) with an activation block: fp32 result
__device__ __forceinline__ int dot_planes(const uint32_t (&wl)[4], const uint32_t (&wh)[4], const int (&x)[8]) {
    int acc = 0;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        acc = __builtin_amdgcn_sdot4(int(wl[q]), x[q], acc, false);
        acc = __builtin_amdgcn_sdot4(int(wh[q]), x[4 + q], acc, false);
    }
    return acc;
}
__device__ __forceinline__ int dot_half(const uint32_t (&w)[4], const int * x) {
    int acc = 0;
#pragma unroll
    for (int q = 0; q < 4; ++q) acc = __builtin_amdgcn_sdot4(int(w[q]), x[q], acc, false);
    return acc;
}

template <uint32_t FMT> struct Sub;

template <> struct Sub<TQMOE_IQ4_XS> {
    static __device__ __forceinline__ float dot(const uint8_t * __restrict__ codes, const uint8_t * __restrict__ aux, int64_t, int, int64_t row,
                                                int S, int s, const ActBlock & x, const uint32_t *) {
        const uint4 c = *reinterpret_cast<const uint4 *>(codes + (row * S + s) * 16);
        const uint2 rec = *reinterpret_cast<const uint2 *>(aux + (row * (S >> 3) + (s >> 3)) * 8);
        const uint32_t w[4] = {c.x, c.y, c.z, c.w};
        uint32_t wl[4], wh[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) lookup16<kIq4T0, kIq4T1, kIq4T2, kIq4T3>(w[q], wl[q], wh[q]);
        const int tot = (dot_planes(wl, wh, x.hi) << 7) + dot_planes(wl, wh, x.lo);
        const float ws = half_bits_to_float(uint16_t(rec.x & 0xFFFFu)) * float(iq4xs_ls(rec, s & 7) - 32);
        return float(tot) * (ws * x.scale);
    }
};

template <> struct Sub<TQMOE_Q4_K> {
    static __device__ __forceinline__ float dot(const uint8_t * __restrict__ codes, const uint8_t * __restrict__ aux, int64_t, int, int64_t row,
                                                int S, int s, const ActBlock & x, const uint32_t *) {
        const uint4 c = *reinterpret_cast<const uint4 *>(codes + (row * S + s) * 16);
        const uint4 rec = *reinterpret_cast<const uint4 *>(aux + (row * (S >> 3) + (s >> 3)) * 16);
        const uint32_t w[4] = {c.x, c.y, c.z, c.w};
        uint32_t wl[4], wh[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) nibbles(w[q], wl[q], wh[q]);
        const int tot = (dot_planes(wl, wh, x.hi) << 7) + dot_planes(wl, wh, x.lo);
        const uint32_t sc12[3] = {rec.y, rec.z, rec.w};
        int sc, mn;
        q4k_scale_min(sc12, s & 7, sc, mn);
        const float d = half_bits_to_float(uint16_t(rec.x & 0xFFFFu)), dmin = half_bits_to_float(uint16_t(rec.x >> 16));
        return float(tot) * (d * float(sc) * x.scale) - dmin * float(mn) * x.sum;
    }
};

template <> struct Sub<TQMOE_NVFP4G> {
    static __device__ __forceinline__ float dot(const uint8_t * __restrict__ codes, const uint8_t * __restrict__ aux, int64_t rows_total, int cols,
                                                int64_t row, int S, int s, const ActBlock & x, const uint32_t *) {
        const uint4 c = *reinterpret_cast<const uint4 *>(codes + (row * S + s) * 16);
        const uint16_t sc = *reinterpret_cast<const uint16_t *>(aux + row * (cols / 16) + 2 * s);
        const float g = *reinterpret_cast<const float *>(aux + nvfp4_global_offset(rows_total, cols) + row * 4);
        const uint32_t w[4] = {c.x, c.y, c.z, c.w};
        uint32_t wl[4], wh[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) lookup16<kFp4T0, kFp4T1, kFp4T2, kFp4T3>(w[q], wl[q], wh[q]);
        // low nibbles = the first 16-weight group, high nibbles = the second; table values are twice the E2M1 value
        const int t0 = (dot_half(wl, x.hi) << 7) + dot_half(wl, x.lo);
        const int t1 = (dot_half(wh, x.hi + 4) << 7) + dot_half(wh, x.lo + 4);
        const float d0 = e4m3_to_float(sc & 0xFFu), d1 = e4m3_to_float(sc >> 8);
        return (float(t0) * d0 + float(t1) * d1) * (0.5f * g * x.scale);
    }
};

template <> struct Sub<TQMOE_IQ3_S> {
    // grid: the 512-entry lattice in LDS
    static __device__ __forceinline__ float dot(const uint8_t * __restrict__ codes, const uint8_t * __restrict__ aux, int64_t, int, int64_t row,
                                                int S, int s, const ActBlock & x, const uint32_t * grid) {
        const uint32_t * cp = reinterpret_cast<const uint32_t *>(codes + (row * S + s) * 12);
        const uint32_t qs[2] = {cp[0], cp[1]}, sg = cp[2];
        const uint4 rec = *reinterpret_cast<const uint4 *>(aux + (row * (S >> 3) + (s >> 3)) * 16);
        const int ib = s & 7;
        const uint32_t qh = ib < 2 ? (rec.x >> (16 + 8 * ib)) & 0xFFu : ib < 6 ? (rec.y >> (8 * (ib - 2))) & 0xFFu : (rec.z >> (8 * (ib - 6))) & 0xFFu;
        const uint32_t scb = (ib >> 1) < 2 ? (rec.z >> (16 + 8 * (ib >> 1))) & 0xFFu : (rec.w >> (8 * ((ib >> 1) - 2))) & 0xFFu;
        int ihi = 0, ilo = 0;
#pragma unroll
        for (int w = 0; w < 8; ++w) {
            const uint32_t g = grid[((qs[w >> 2] >> (8 * (w & 3))) & 0xFFu) | (((qh >> w) & 1u) << 8)];
            // four sign bits -> byte masks 0xFF; negate the selected bytes: (g ^ m) + (m & 0x01010101), no carry leaves a byte
            const uint32_t bits = (((sg >> (4 * w)) & 15u) * 0x00204081u) & 0x01010101u;
            const uint32_t m = (bits << 8) - bits;
            const uint32_t sv = (g ^ m) + bits;
            ihi = __builtin_amdgcn_sdot4(int(sv), x.hi[w], ihi, false);
            ilo = __builtin_amdgcn_sdot4(int(sv), x.lo[w], ilo, false);
        }
        const float db = half_bits_to_float(uint16_t(rec.x & 0xFFFFu)) * float(1 + 2 * int((scb >> (4 * (ib & 1))) & 15u));
        return float((ihi << 7) + ilo) * (db * x.scale);
    }
};

template <uint32_t FMT> __device__ __forceinline__ const uint32_t * stage_grid(uint32_t * lds) {
    if constexpr (FMT == TQMOE_IQ3_S) {
        for (int i = threadIdx.x; i < 512; i += blockDim.x) lds[i] = d_iq3s_grid.v[i];
        __syncthreads();
        return lds;
    } else {
        return nullptr;
    }
}

struct BankView { const uint8_t * codes; const uint8_t * aux; int64_t rows_total; int rows, cols; };
inline BankView view(const tqmoe_bank & b) {
    return BankView{static_cast<const uint8_t *>(b.codes), static_cast<const uint8_t *>(b.aux), int64_t(b.experts) * b.rows, b.rows, b.cols};
}

// lanes per row and sub-blocks per lane for S sub-blocks per row
struct Split { int lpr, m; };
inline Split split_for(int S) {
    if (S % 64 == 0) return Split{64, S / 64};
    int lpr = 1;
    while (lpr < 32 && S % (lpr * 2) == 0) lpr *= 2;
    if (S / lpr <= 4) return Split{lpr, S / lpr};
    lpr = 64;  // ragged: lanes past the row's last sub-block idle
    while (lpr / 2 >= S) lpr /= 2;
    return Split{lpr, (S + lpr - 1) / lpr};
}

// one row of the stacked matrix times the lane's activation blocks; sub-blocks s >= s_end contribute nothing
template <uint32_t FMT, int M>
__device__ __forceinline__ float row_dot(const BankView & b, int64_t row, int S, int sl, int lpr, int s_end, const ActBlock (&x)[M], const uint32_t * grid) {
    float acc = 0.f;
#pragma unroll
    for (int m = 0; m < M; ++m) {
        const int s = sl + lpr * m;
        const float v = Sub<FMT>::dot(b.codes, b.aux, b.rows_total, b.cols, row, S, min(s, S - 1), x[m], grid);
        acc += s < s_end ? v : 0.f;
    }
    return acc;
}

// ------------------------------------------------------------------------------------------- grouped mat-vec
// grid (row tiles, assignments). y[a][r] for the tile's rows; NB banks (gate and up) share ids and the input image.
template <uint32_t FMT, int M, int NB>
__global__ __launch_bounds__(256) void matvec_k(BankView b0, BankView b1, const uint8_t * __restrict__ image, void * y0, void * y1, uint32_t ytype,
                                                const int * __restrict__ ids, int topk, int per_expert_input, int lpr, int iters) {
    __shared__ uint32_t grid_lds[FMT == TQMOE_IQ3_S ? 512 : 1];
    const uint32_t * grid = stage_grid<FMT>(grid_lds);
    const int a = blockIdx.y;
    const int e = ids[a];
    if (e < 0) return;
    const int S = b0.cols / 32, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int rw = 64 / lpr, rl = lane / lpr, sl = lane % lpr;
    const uint8_t * image_row = image + int64_t(per_expert_input ? a : a / topk) * S * kImageSubBytes;
    ActBlock x[M];
#pragma unroll
    for (int m = 0; m < M; ++m) {
        const int s = sl + lpr * m;
        if (s < S) load_act_block(image_row, S, s, x[m]); else zero_act_block(x[m]);
    }
    const int tile0 = blockIdx.x * (4 * rw * iters);
    for (int it = 0; it < iters; ++it) {
        const int r = tile0 + (it * 4 + wave) * rw + rl;
        const int rc = min(r, b0.rows - 1);
        const int64_t row = int64_t(e) * b0.rows + rc;
        float v0 = row_dot<FMT, M>(b0, row, S, sl, lpr, S, x, grid);
        float v1 = 0.f;
        if constexpr (NB == 2) v1 = row_dot<FMT, M>(b1, row, S, sl, lpr, S, x, grid);
        v0 = group_sum_rt(v0, lpr);
        if constexpr (NB == 2) v1 = group_sum_rt(v1, lpr);
        if (sl == 0 && r < b0.rows) {
            const int64_t o = int64_t(a) * b0.rows + r;
            if (ytype == TQMOE_F32) { static_cast<float *>(y0)[o] = v0; if constexpr (NB == 2) static_cast<float *>(y1)[o] = v1; }
            else { static_cast<uint16_t *>(y0)[o] = float_to_bf16_bits(v0); if constexpr (NB == 2) static_cast<uint16_t *>(y1)[o] = float_to_bf16_bits(v1); }
        }
    }
}

// ------------------------------------------------------------------------- fused gate + up + SwiGLU (layer path)
// grid (ff / 32, n * slots): one block makes one 32-value sub-block of act = silu(gate x) * (up x) for one
// assignment and writes it straight into the activation image the down product reads. slots = topk (+ 1 for the
// shared expert, which is expert index n_expert and only has shared_ff rows).
template <uint32_t FMT, int M>
__global__ __launch_bounds__(256) void gateup_k(BankView bg, BankView bu, const uint8_t * __restrict__ ximage, uint8_t * __restrict__ aimage,
                                                const int * __restrict__ ids, int topk, int slots, int n_expert, int shared_ff, int lpr) {
    __shared__ uint32_t grid_lds[FMT == TQMOE_IQ3_S ? 512 : 1];
    __shared__ float gl[32], ul[32];
    const uint32_t * grid = stage_grid<FMT>(grid_lds);
    const int a = blockIdx.y, t = a / slots, sl_ot = a % slots;
    const int e = sl_ot < topk ? ids[t * topk + sl_ot] : n_expert;
    const int ff_here = sl_ot < topk ? bg.rows : shared_ff;
    const int tile0 = blockIdx.x * 32;
    if (e < 0 || tile0 >= ff_here) return;
    const int S = bg.cols / 32, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int rw = 64 / lpr, rl = lane / lpr, sl = lane % lpr;
    const uint8_t * image_row = ximage + int64_t(t) * S * kImageSubBytes;
    ActBlock x[M];
#pragma unroll
    for (int m = 0; m < M; ++m) {
        const int s = sl + lpr * m;
        if (s < S) load_act_block(image_row, S, s, x[m]); else zero_act_block(x[m]);
    }
    for (int r0 = wave * rw; r0 < 32; r0 += 4 * rw) {
        const int r = r0 + rl;  // past 31 only when a wave spans more than 32 rows: computed on row 31, not stored
        const int64_t row = int64_t(e) * bg.rows + tile0 + min(r, 31);
        float g = row_dot<FMT, M>(bg, row, S, sl, lpr, S, x, grid);
        float u = row_dot<FMT, M>(bu, row, S, sl, lpr, S, x, grid);
        g = group_sum_rt(g, lpr);
        u = group_sum_rt(u, lpr);
        if (sl == 0 && r < 32) { gl[r] = g; ul[r] = u; }
    }
    __syncthreads();
    if (threadIdx.x == 0) {  // 32 values: one lane quantises the block
        float v[32];
#pragma unroll
        for (int i = 0; i < 32; ++i) { const float g = gl[i]; v[i] = g / (1.f + expf(-g)) * ul[i]; }
        const int SA = bg.rows / 32;
        uint8_t * base = aimage + int64_t(a) * SA * kImageSubBytes;
        quantise_block(v, base + int64_t(blockIdx.x) * 64, base + int64_t(SA) * 64 + int64_t(blockIdx.x) * 8);
    }
}

// ------------------------------------------------------------------------------ fused down + combine (layer path)
// grid (row tiles, tokens). out[t][r] = sum over slots in order of weight * (down_e(slot) act(slot)), the shared
// expert last with sigmoid weight; each lane keeps its partial sums in slot order and the butterfly runs once.
template <uint32_t FMT, int M, int OT>
__global__ void down_combine_k(BankView bd, const uint8_t * __restrict__ aimage, const int * __restrict__ ids, const float * __restrict__ weights,
                               const float * __restrict__ shared_w, void * __restrict__ out, int topk, int slots, int n_expert, int shared_ff, int lpr) {
    __shared__ uint32_t grid_lds[FMT == TQMOE_IQ3_S ? 512 : 1];
    const uint32_t * grid = stage_grid<FMT>(grid_lds);
    const int t = blockIdx.y;
    const int S = bd.cols / 32, lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
    const int rw = 64 / lpr, rl = lane / lpr, sl = lane % lpr;
    const int r = (blockIdx.x * waves + wave) * rw + rl;
    const int rc = min(r, bd.rows - 1);
    float acc = 0.f;
    for (int so = 0; so < slots; ++so) {
        const int e = so < topk ? ids[t * topk + so] : n_expert;
        if (e < 0) continue;
        const float wgt = so < topk ? weights[t * topk + so] : shared_w[t];
        const int s_end = so < topk ? S : shared_ff / 32;
        const uint8_t * image_row = aimage + (int64_t(t) * slots + so) * S * kImageSubBytes;
        ActBlock x[M];
#pragma unroll
        for (int m = 0; m < M; ++m) {
            const int s = sl + lpr * m;
            if (s < s_end) load_act_block(image_row, S, s, x[m]); else zero_act_block(x[m]);
        }
        acc += wgt * row_dot<FMT, M>(bd, int64_t(e) * bd.rows + rc, S, sl, lpr, s_end, x, grid);
    }
    acc = group_sum_rt(acc, lpr);
    if (sl == 0 && r < bd.rows) store_out<OT>(out, int64_t(t) * bd.rows + r, acc);
}

// ------------------------------------------------------------------------------------------ elementwise helpers
__global__ __launch_bounds__(256) void swiglu_k(const float * __restrict__ g, const float * __restrict__ u, float * __restrict__ act, int64_t count) {
    const int64_t i = int64_t(blockIdx.x) * 256 + threadIdx.x;
    if (i < count) { const float a = g[i]; act[i] = a / (1.f + expf(-a)) * u[i]; }
}

template <int OT>
__global__ __launch_bounds__(256) void combine_k(const float * __restrict__ routed, const float * __restrict__ shared, const float * __restrict__ weights,
                                                 const float * __restrict__ shared_w, void * __restrict__ out, int h, int k, int64_t count) {
    const int64_t i = int64_t(blockIdx.x) * 256 + threadIdx.x;
    if (i >= count) return;
    const int64_t t = i / h;
    const int j = int(i % h);
    float sum = 0.f;
    for (int s = 0; s < k; ++s) sum += weights[t * k + s] * routed[(t * k + s) * h + j];
    if (shared) sum += shared_w[t] * shared[i];
    store_out<OT>(out, i, sum);
}

// --------------------------------------------------------------------------------------------------- launchers
template <uint32_t FMT, int NB>
void launch_matvec(int m, dim3 grid, hipStream_t s, BankView b0, BankView b1, const uint8_t * image, void * y0, void * y1, uint32_t ytype,
                   const int * ids, int topk, int pei, int lpr, int iters) {
    switch (m) {
        case 1: matvec_k<FMT, 1, NB><<<grid, 256, 0, s>>>(b0, b1, image, y0, y1, ytype, ids, topk, pei, lpr, iters); break;
        case 2: matvec_k<FMT, 2, NB><<<grid, 256, 0, s>>>(b0, b1, image, y0, y1, ytype, ids, topk, pei, lpr, iters); break;
        case 3: matvec_k<FMT, 3, NB><<<grid, 256, 0, s>>>(b0, b1, image, y0, y1, ytype, ids, topk, pei, lpr, iters); break;
        default: matvec_k<FMT, 4, NB><<<grid, 256, 0, s>>>(b0, b1, image, y0, y1, ytype, ids, topk, pei, lpr, iters); break;
    }
}
template <int NB>
void launch_matvec_fmt(uint32_t fmt, int m, dim3 grid, hipStream_t s, BankView b0, BankView b1, const uint8_t * image, void * y0, void * y1,
                       uint32_t ytype, const int * ids, int topk, int pei, int lpr, int iters) {
    switch (fmt) {
        case TQMOE_IQ4_XS: launch_matvec<TQMOE_IQ4_XS, NB>(m, grid, s, b0, b1, image, y0, y1, ytype, ids, topk, pei, lpr, iters); break;
        case TQMOE_Q4_K: launch_matvec<TQMOE_Q4_K, NB>(m, grid, s, b0, b1, image, y0, y1, ytype, ids, topk, pei, lpr, iters); break;
        case TQMOE_IQ3_S: launch_matvec<TQMOE_IQ3_S, NB>(m, grid, s, b0, b1, image, y0, y1, ytype, ids, topk, pei, lpr, iters); break;
        default: launch_matvec<TQMOE_NVFP4G, NB>(m, grid, s, b0, b1, image, y0, y1, ytype, ids, topk, pei, lpr, iters); break;
    }
}

template <uint32_t FMT>
void launch_gateup(int m, dim3 grid, hipStream_t s, BankView bg, BankView bu, const uint8_t * ximage, uint8_t * aimage, const int * ids, int topk,
                   int slots, int n_expert, int shared_ff, int lpr) {
    switch (m) {
        case 1: gateup_k<FMT, 1><<<grid, 256, 0, s>>>(bg, bu, ximage, aimage, ids, topk, slots, n_expert, shared_ff, lpr); break;
        case 2: gateup_k<FMT, 2><<<grid, 256, 0, s>>>(bg, bu, ximage, aimage, ids, topk, slots, n_expert, shared_ff, lpr); break;
        case 3: gateup_k<FMT, 3><<<grid, 256, 0, s>>>(bg, bu, ximage, aimage, ids, topk, slots, n_expert, shared_ff, lpr); break;
        default: gateup_k<FMT, 4><<<grid, 256, 0, s>>>(bg, bu, ximage, aimage, ids, topk, slots, n_expert, shared_ff, lpr); break;
    }
}

template <uint32_t FMT, int OT>
void launch_down(int m, dim3 grid, int threads, hipStream_t s, BankView bd, const uint8_t * aimage, const int * ids, const float * weights,
                 const float * shared_w, void * out, int topk, int slots, int n_expert, int shared_ff, int lpr) {
    switch (m) {
        case 1: down_combine_k<FMT, 1, OT><<<grid, threads, 0, s>>>(bd, aimage, ids, weights, shared_w, out, topk, slots, n_expert, shared_ff, lpr); break;
        case 2: down_combine_k<FMT, 2, OT><<<grid, threads, 0, s>>>(bd, aimage, ids, weights, shared_w, out, topk, slots, n_expert, shared_ff, lpr); break;
        case 3: down_combine_k<FMT, 3, OT><<<grid, threads, 0, s>>>(bd, aimage, ids, weights, shared_w, out, topk, slots, n_expert, shared_ff, lpr); break;
        default: down_combine_k<FMT, 4, OT><<<grid, threads, 0, s>>>(bd, aimage, ids, weights, shared_w, out, topk, slots, n_expert, shared_ff, lpr); break;
    }
}

}  // namespace

// used by the whole-layer entry point (layer.hip)
int32_t enqueue_quant_act(const void * x, uint32_t xtype, int n, int cols, void * image, hipStream_t s) {
    const int64_t subs = int64_t(n) * (cols / 32);
    const unsigned blocks = unsigned((subs + 255) / 256);
    switch (xtype) {
        case TQMOE_F32: quant_act_k<TQMOE_F32><<<blocks, 256, 0, s>>>(x, n, cols, static_cast<uint8_t *>(image)); break;
        case TQMOE_F16: quant_act_k<TQMOE_F16><<<blocks, 256, 0, s>>>(x, n, cols, static_cast<uint8_t *>(image)); break;
        default: quant_act_k<TQMOE_BF16><<<blocks, 256, 0, s>>>(x, n, cols, static_cast<uint8_t *>(image)); break;
    }
    return 0;
}

}  // namespace tqmoe

using namespace tqmoe;

extern "C" int32_t tqmoe_expert_gateup(const tqmoe_bank * gate, const tqmoe_bank * up, const void * x_image, void * act_image, const int32_t * ids,
                                       int32_t n, int32_t topk, int32_t has_shared, int32_t shared_ff, void * stream, tqmoe_error * err) {
    const char * what = "tqmoe_expert_gateup";
    if (int32_t rc = check_bank(gate, what, err)) return rc;
    if (int32_t rc = check_bank(up, what, err)) return rc;
    if (up->type != gate->type || up->rows != gate->rows || up->cols != gate->cols || up->experts != gate->experts)
        return fail(err, TQMOE_E_ARG, "%s: the two banks differ in format or shape", what);
    if (!x_image || !act_image || !ids || n <= 0 || topk <= 0 || gate->rows % 32) return fail(err, TQMOE_E_ARG, "%s: invalid shape or pointer", what);
    if (has_shared && (shared_ff <= 0 || shared_ff > gate->rows || shared_ff % 32)) return fail(err, TQMOE_E_ARG, "%s: invalid shared_ff", what);
    const int slots = topk + (has_shared ? 1 : 0), n_expert = gate->experts - (has_shared ? 1 : 0);
    if (n_expert <= 0 || int64_t(n) * slots > 65535) return fail(err, TQMOE_E_ARG, "%s: n * slots exceeds 65535 or the bank is too small", what);
    const Split sp = split_for(gate->cols / 32);
    if (sp.m > 4) return fail(err, TQMOE_E_UNSUPPORTED, "%s: cols %d is too wide for the decode kernels", what, gate->cols);
    if (int32_t rc = need_device(err, what)) return rc;
    const hipStream_t s = static_cast<hipStream_t>(stream);
    const dim3 grid(unsigned(gate->rows / 32), unsigned(n * slots));
    const BankView bg = view(*gate), bu = view(*up);
    const uint8_t * xi = static_cast<const uint8_t *>(x_image);
    uint8_t * ai = static_cast<uint8_t *>(act_image);
    switch (gate->type) {
        case TQMOE_IQ4_XS: launch_gateup<TQMOE_IQ4_XS>(sp.m, grid, s, bg, bu, xi, ai, ids, topk, slots, n_expert, shared_ff, sp.lpr); break;
        case TQMOE_Q4_K: launch_gateup<TQMOE_Q4_K>(sp.m, grid, s, bg, bu, xi, ai, ids, topk, slots, n_expert, shared_ff, sp.lpr); break;
        case TQMOE_IQ3_S: launch_gateup<TQMOE_IQ3_S>(sp.m, grid, s, bg, bu, xi, ai, ids, topk, slots, n_expert, shared_ff, sp.lpr); break;
        default: launch_gateup<TQMOE_NVFP4G>(sp.m, grid, s, bg, bu, xi, ai, ids, topk, slots, n_expert, shared_ff, sp.lpr); break;
    }
    return launched(err, what);
}

extern "C" int32_t tqmoe_expert_down_combine(const tqmoe_bank * down, const void * act_image, const int32_t * ids, const float * weights,
                                             const float * shared_weights, void * out, uint32_t otype, int32_t n, int32_t topk, int32_t has_shared,
                                             int32_t shared_ff, void * stream, tqmoe_error * err) {
    const char * what = "tqmoe_expert_down_combine";
    if (int32_t rc = check_bank(down, what, err)) return rc;
    if (!act_image || !ids || !weights || !out || n <= 0 || topk <= 0 || (has_shared && !shared_weights)) return fail(err, TQMOE_E_ARG, "%s: invalid shape or pointer", what);
    if (has_shared && (shared_ff <= 0 || shared_ff > down->cols || shared_ff % 32)) return fail(err, TQMOE_E_ARG, "%s: invalid shared_ff", what);
    if (otype != TQMOE_F32 && otype != TQMOE_BF16) return fail(err, TQMOE_E_UNSUPPORTED, "%s: output type must be F32 or BF16", what);
    const int slots = topk + (has_shared ? 1 : 0), n_expert = down->experts - (has_shared ? 1 : 0);
    if (n_expert <= 0 || n > 65535) return fail(err, TQMOE_E_ARG, "%s: too many tokens for one call or the bank is too small", what);
    const Split sp = split_for(down->cols / 32);
    if (sp.m > 4) return fail(err, TQMOE_E_UNSUPPORTED, "%s: cols %d is too wide for the decode kernels", what, down->cols);
    if (int32_t rc = need_device(err, what)) return rc;
    const hipStream_t s = static_cast<hipStream_t>(stream);
    const int rw = 64 / sp.lpr;
    // few tokens: one wave per block so that the grid still covers the chip
    const int waves = int64_t(n) * ((down->rows + rw - 1) / rw) >= 4096 ? 4 : 1;
    const dim3 grid(unsigned((down->rows + rw * waves - 1) / (rw * waves)), unsigned(n));
    const BankView bd = view(*down);
    const uint8_t * ai = static_cast<const uint8_t *>(act_image);
#define TQ_DOWN(F)                                                                                                                              \
    if (otype == TQMOE_F32) launch_down<F, TQMOE_F32>(sp.m, grid, waves * 64, s, bd, ai, ids, weights, shared_weights, out, topk, slots, n_expert, shared_ff, sp.lpr); \
    else launch_down<F, TQMOE_BF16>(sp.m, grid, waves * 64, s, bd, ai, ids, weights, shared_weights, out, topk, slots, n_expert, shared_ff, sp.lpr)
    switch (down->type) {
        case TQMOE_IQ4_XS: TQ_DOWN(TQMOE_IQ4_XS); break;
        case TQMOE_Q4_K: TQ_DOWN(TQMOE_Q4_K); break;
        case TQMOE_IQ3_S: TQ_DOWN(TQMOE_IQ3_S); break;
        default: TQ_DOWN(TQMOE_NVFP4G); break;
    }
#undef TQ_DOWN
    return launched(err, what);
}

extern "C" size_t tqmoe_act_image_bytes(int32_t n, int32_t cols) {
    if (n <= 0 || cols <= 0 || cols % 32) return 0;
    return size_t(n) * size_t(cols / 32) * kImageSubBytes;
}

extern "C" int32_t tqmoe_quant_act(const void * x, uint32_t xtype, int32_t n, int32_t cols, void * image, void * stream, tqmoe_error * err) {
    if (!x || !image || n <= 0 || cols <= 0 || cols % 32) return fail(err, TQMOE_E_ARG, "tqmoe_quant_act: invalid shape or pointer (cols must be a multiple of 32)");
    if (!is_act_type(xtype)) return fail(err, TQMOE_E_UNSUPPORTED, "tqmoe_quant_act: unsupported element type");
    if (int32_t rc = need_device(err, "tqmoe_quant_act")) return rc;
    enqueue_quant_act(x, xtype, n, cols, image, static_cast<hipStream_t>(stream));
    return launched(err, "tqmoe_quant_act");
}

static int32_t matvec_common(const tqmoe_bank * b0, const tqmoe_bank * b1, const void * image, void * y0, void * y1, uint32_t ytype,
                             const int32_t * ids, int32_t n, int32_t topk, int32_t pei, void * stream, tqmoe_error * err, const char * what) {
    if (int32_t rc = check_bank(b0, what, err)) return rc;
    if (b1) {
        if (int32_t rc = check_bank(b1, what, err)) return rc;
        if (b1->type != b0->type || b1->rows != b0->rows || b1->cols != b0->cols || b1->experts != b0->experts)
            return fail(err, TQMOE_E_ARG, "%s: the two banks differ in format or shape", what);
    }
    if (!image || !y0 || (b1 && !y1) || !ids || n <= 0 || topk <= 0) return fail(err, TQMOE_E_ARG, "%s: invalid shape or pointer", what);
    if (int64_t(n) * topk > 65535) return fail(err, TQMOE_E_ARG, "%s: n * topk exceeds 65535", what);  // src/formats/weight/quant.cu:73
    if (ytype != TQMOE_F32 && ytype != TQMOE_BF16) return fail(err, TQMOE_E_UNSUPPORTED, "%s: output type must be F32 or BF16", what);
    const Split sp = split_for(b0->cols / 32);
    if (sp.m > 4) return fail(err, TQMOE_E_UNSUPPORTED, "%s: cols %d is too wide for the decode kernels", what, b0->cols);
    if (int32_t rc = need_device(err, what)) return rc;
    const int rw = 64 / sp.lpr;
    const int iters = int64_t(n) * topk * ((b0->rows + 4 * rw - 1) / (4 * rw)) >= 8192 ? 4 : 1;
    const dim3 grid(unsigned((b0->rows + 4 * rw * iters - 1) / (4 * rw * iters)), unsigned(n * topk));
    const hipStream_t s = static_cast<hipStream_t>(stream);
    const BankView v0 = view(*b0), v1 = b1 ? view(*b1) : v0;
    if (b1) launch_matvec_fmt<2>(b0->type, sp.m, grid, s, v0, v1, static_cast<const uint8_t *>(image), y0, y1, ytype, ids, topk, pei, sp.lpr, iters);
    else launch_matvec_fmt<1>(b0->type, sp.m, grid, s, v0, v1, static_cast<const uint8_t *>(image), y0, y1, ytype, ids, topk, pei, sp.lpr, iters);
    return launched(err, what);
}

extern "C" int32_t tqmoe_expert_matvec(const tqmoe_bank * bank, const void * image, void * y, uint32_t ytype, const int32_t * ids, int32_t n,
                                       int32_t topk, int32_t per_expert_input, void * stream, tqmoe_error * err) {
    return matvec_common(bank, nullptr, image, y, nullptr, ytype, ids, n, topk, per_expert_input, stream, err, "tqmoe_expert_matvec");
}

extern "C" int32_t tqmoe_expert_matvec2(const tqmoe_bank * gate, const tqmoe_bank * up, const void * image, void * y_gate, void * y_up, uint32_t ytype,
                                        const int32_t * ids, int32_t n, int32_t topk, void * stream, tqmoe_error * err) {
    if (!up) return fail(err, TQMOE_E_ARG, "tqmoe_expert_matvec2: second bank missing");
    return matvec_common(gate, up, image, y_gate, y_up, ytype, ids, n, topk, 0, stream, err, "tqmoe_expert_matvec2");
}

extern "C" int32_t tqmoe_swiglu(const float * gate, const float * up, float * act, int64_t count, void * stream, tqmoe_error * err) {
    if (!gate || !up || !act || count <= 0 || (count + 255) / 256 > 0x7FFFFFFF) return fail(err, TQMOE_E_ARG, "tqmoe_swiglu: invalid size or pointer");
    if (int32_t rc = need_device(err, "tqmoe_swiglu")) return rc;
    swiglu_k<<<unsigned((count + 255) / 256), 256, 0, static_cast<hipStream_t>(stream)>>>(gate, up, act, count);
    return launched(err, "tqmoe_swiglu");
}

extern "C" int32_t tqmoe_combine(const float * routed, const float * shared, const float * weights, const float * shared_weights, void * out,
                                 uint32_t otype, int32_t hidden, int32_t topk, int32_t n, void * stream, tqmoe_error * err) {
    if (!routed || !weights || !out || hidden <= 0 || topk <= 0 || n <= 0 || (shared && !shared_weights))
        return fail(err, TQMOE_E_ARG, "tqmoe_combine: invalid shape or pointer");
    if (otype != TQMOE_F32 && otype != TQMOE_BF16) return fail(err, TQMOE_E_UNSUPPORTED, "tqmoe_combine: output type must be F32 or BF16");
    if (int32_t rc = need_device(err, "tqmoe_combine")) return rc;
    const int64_t count = int64_t(n) * hidden;
    const unsigned blocks = unsigned((count + 255) / 256);
    const hipStream_t s = static_cast<hipStream_t>(stream);
    if (otype == TQMOE_F32) combine_k<TQMOE_F32><<<blocks, 256, 0, s>>>(routed, shared, weights, shared_weights, out, hidden, topk, count);
    else combine_k<TQMOE_BF16><<<blocks, 256, 0, s>>>(routed, shared, weights, shared_weights, out, hidden, topk, count);
    return launched(err, "tqmoe_combine");
}

// Prefill-sized expert products of any bank format: a grouped fp16 x fp16 -> fp32 GEMM on the matrix pipe (the kernels;
// prefill_f16.hip holds the entry, and one translation unit per bank format instantiates F16Launch<FMT>).
//
// The counterpart of the reference's WeightFormat::expert_gemm / expert_gemm_gateup (weight_format.hpp:51-59): weights
// turned into fp16 operands in registers, input rows converted to fp16 tiles in LDS, products accumulated in fp32 by
// v_mfma_f32_32x32x16_f16, gate and up in one launch with the SwiGLU epilogue.
//
// A block takes one expert, up to 128 (or 64) of its assignments (the dispatch lists give them) and 128 weight rows of
// each bank; each of its four waves owns 32 of the weight rows and all the block's input rows, four (two) 32 x 32 tiles per
// bank. Per stage of 64 weights of a row, lane (r, g) of a wave decodes sub-block g of its weight row r: those sixteen
// dwords ARE its weight operands of the stage's four matrix instructions per tile, so weights never pass through LDS.
// The input tile does (double-buffered, one barrier per stage), each 16-byte operand read feeding one instruction per
// bank. Weight and input loads are issued one stage ahead of their use.
//
// Weight values. A thread takes one 32-weight sub-block through the format's decode-kernel traits (Sub<FMT>: the int8
// values q, the scale(s) and the minimum(s)) and makes fp16(q * scale - minimum) with one fp32 multiply-add per weight:
// the product and the difference are rounded once in fp32 (2^-24) and once to fp16, where the exact decoder of the
// fp32 dequantiser rounds them separately; the difference is far below the fp16 step.
#pragma once
#include "decode_kernels.cuh"

namespace tqmoe {
namespace {

typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef _Float16 v2h __attribute__((ext_vector_type(2)));
typedef float v16f __attribute__((ext_vector_type(16)));

// the expert whose run of ROWS-row blocks holds `unit`; local = the block inside the expert; expert = -1 past the last
struct Where { int expert, local; };
template <int ROWS> __device__ __forceinline__ Where locate(const int * __restrict__ counts, int experts, int unit) {
    __shared__ Where w;
    if (threadIdx.x < 64) {
        const int lane = threadIdx.x;
        if (lane == 0) w.expert = -1;
        int base = 0;
        for (int e0 = 0; e0 < experts; e0 += 64) {
            const int e = e0 + lane;
            const int units = e < experts ? (max(counts[e], 0) + ROWS - 1) / ROWS : 0;
            int ui = units;
#pragma unroll
            for (int d = 1; d < 64; d <<= 1) { const int a = __shfl_up(ui, d, 64); if (lane >= d) ui += a; }
            if (units > 0 && unit >= base + ui - units && unit < base + ui) { w.expert = e; w.local = unit - (base + ui - units); }
            base += __shfl(ui, 63, 64);
            if (unit < base) break;
        }
    }
    __syncthreads();
    return w;
}

typedef float v2f __attribute__((ext_vector_type(2)));
// two floats -> two halves, round to nearest even (one packed conversion)
__device__ __forceinline__ uint32_t pack_h2(float a, float b) {
    const v2f v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, v2h));
}

// four int8 values -> four halves fp16(q * scale - minimum) (two dwords): the bytes are biased to unsigned so that each
// converts to fp32 in one instruction, and the bias goes into the constant of the multiply-add, c = -(128 scale + minimum)
__device__ __forceinline__ uint2 i8x4_to_h4(uint32_t w, float scale, float c) {
    const uint32_t u = w ^ 0x80808080u;
    const float f0 = float(u & 0xFFu), f1 = float((u >> 8) & 0xFFu), f2 = float((u >> 16) & 0xFFu), f3 = float(u >> 24);
    return make_uint2(pack_h2(fmaf(f0, scale, c), fmaf(f1, scale, c)), pack_h2(fmaf(f2, scale, c), fmaf(f3, scale, c)));
}

// The fp16 values of sub-block s of weight row `row` (an index into the stacked bank), as 16 dwords in weight order, in two
// steps so that the loads of a stage can be in flight during the products of the one before: load() issues the loads,
// finish() turns what they brought into halves.
template <uint32_t FMT> struct F16Sub {
    typedef typename Sub<FMT>::Raw Raw;
    static __device__ __forceinline__ Raw load(const BankView & b, int64_t row, int s) {
        Tile t;
        t.codes = b.codes + row * code_row_bytes(FMT, b.cols);
        t.aux = b.aux + row * aux_row_bytes(FMT, b.cols);
        t.aux2 = FMT == TQMOE_NVFP4G ? b.aux + nvfp4_global_offset(b.rows_total, b.cols) + row * 4 : nullptr;
        return Sub<FMT>::load(t, 0u, uint32_t(b.cols / 32), uint32_t(s));
    }
    // valid false: all zeros (a row or a sub-block past the end), through a zero scale and constant
    static __device__ __forceinline__ void finish(const Raw & raw, int s, const uint32_t * grid, bool valid, uint32_t (&h)[16]) {
        Dec d;
        d.mn1 = 0.f;
        Sub<FMT>::decode(raw, s, grid, d);
        const float s0 = valid ? d.s0 : 0.f, s1 = valid ? d.s1 : 0.f;
        const float c0 = valid ? -(128.f * d.s0 + d.mn) : 0.f, c1 = valid ? -(128.f * d.s1 + (HalfMins<Sub<FMT>>::value ? d.mn1 : d.mn)) : 0.f;
#pragma unroll
        for (int q = 0; q < 8; ++q) {
            const uint2 v = i8x4_to_h4(d.w[q], q < 4 ? s0 : s1, q < 4 ? c0 : c1);
            h[2 * q] = v.x;
            h[2 * q + 1] = v.y;
        }
    }
};
// IQ4_XS banks are tile-major and have kernels of their own for the decode-sized products: the same steps from the
// tile-major offsets
template <> struct F16Sub<TQMOE_IQ4_XS> {
    struct Raw { uint4 c; uint2 rec; };
    static __device__ __forceinline__ Raw load(const BankView & b, int64_t row, int s) {
        const int S = b.cols / 32;
        Raw r;
        r.c = *reinterpret_cast<const uint4 *>(b.codes + iq4xs_code_offset(row, S, s));
        r.rec = *reinterpret_cast<const uint2 *>(b.aux + iq4xs_aux_offset(row, S, s / 8));
        return r;
    }
    static __device__ __forceinline__ void finish(const Raw & r, int s, const uint32_t *, bool valid, uint32_t (&h)[16]) {
        const float sc = valid ? half_bits_to_float(iq4xs_d_bits(r.rec)) * float(iq4xs_lsm32(r.rec, s & 7)) : 0.f, c0 = -128.f * sc;
        const uint32_t w[4] = {r.c.x, r.c.y, r.c.z, r.c.w};
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            uint32_t lo, hi;
            lookup16<kIq4T0, kIq4T1, kIq4T2, kIq4T3>(w[q], lo, hi);
            const uint2 a = i8x4_to_h4(lo, sc, c0), z = i8x4_to_h4(hi, sc, c0);
            h[2 * q] = a.x; h[2 * q + 1] = a.y;
            h[8 + 2 * q] = z.x; h[8 + 2 * q + 1] = z.y;
        }
    }
};

// 32 input values of a row: 16-bit types are fetched a stage ahead as four 16-byte pieces, fp32 rows at the time of use
struct RawX { uint4 v[4]; };
__device__ __forceinline__ RawX load_x32(const void * x, uint32_t xtype, int64_t at) {
    RawX r;
    if (xtype != TQMOE_F32) {
#pragma unroll
        for (int q = 0; q < 4; ++q) r.v[q] = reinterpret_cast<const uint4 *>(static_cast<const uint16_t *>(x) + at)[q];
    } else {
#pragma unroll
        for (int q = 0; q < 4; ++q) r.v[q] = make_uint4(0u, 0u, 0u, 0u);
    }
    return r;
}
__device__ __forceinline__ void finish_x32(const RawX & r, const void * x, uint32_t xtype, int64_t at, uint32_t (&h)[16]) {
    if (xtype == TQMOE_F16) {
#pragma unroll
        for (int q = 0; q < 4; ++q) { h[4 * q] = r.v[q].x; h[4 * q + 1] = r.v[q].y; h[4 * q + 2] = r.v[q].z; h[4 * q + 3] = r.v[q].w; }
    } else if (xtype == TQMOE_BF16) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const uint32_t w[4] = {r.v[q].x, r.v[q].y, r.v[q].z, r.v[q].w};
#pragma unroll
            for (int j = 0; j < 4; ++j) h[4 * q + j] = pack_h2(__uint_as_float(w[j] << 16), __uint_as_float(w[j] & 0xFFFF0000u));
        }
    } else {
        float v[8];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            load8<TQMOE_F32>(x, at + q * 8, v);
#pragma unroll
            for (int j = 0; j < 4; ++j) h[4 * q + j] = pack_h2(v[2 * j], v[2 * j + 1]);
        }
    }
}

template <uint32_t FMT, int NB, int MT>
__global__ __launch_bounds__(256, 2) void expert_gemm_f16_k(F16Args k) {
    constexpr int kM = 32 * MT, kN = 128, kK = 64, kPad = kK + 8;   // padded rows: 16-byte reads of consecutive rows spread over the LDS banks
    __shared__ __attribute__((aligned(16))) uint16_t As[2][kM][kPad];
    __shared__ __attribute__((aligned(8))) uint32_t grid_lds[lattice_dwords(FMT)];
    __shared__ int s_asg[kM];
    const Where w = locate<kM>(k.counts, k.experts, int(blockIdx.y));
    const int e = w.expert;
    if (e < 0) return;
    const uint32_t * grid = stage_grid<FMT>(grid_lds);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, r = lane & 31, g = lane >> 5;
    const BankView & b0 = k.b0;
    const int rows = b0.rows, cols = b0.cols, S = cols / 32, row0 = int(blockIdx.x) * kN;
    const bool is_shared = e == k.shared_expert;
    const int row_lim = k.gateup && is_shared ? k.shared_lim : rows;     // weight rows this expert has
    const int s_end = !k.gateup && is_shared ? k.shared_lim / 32 : S;    // sub-blocks of the input rows it reads
    const int cnt = k.counts[e], first = w.local * kM;
    if (tid < kM) s_asg[tid] = first + tid < cnt ? k.perm[k.offsets[e] + first + tid] : -1;
    for (int i = tid; i < 2 * kM * kPad / 8; i += 256) reinterpret_cast<uint4 *>(&As[0][0][0])[i] = make_uint4(0u, 0u, 0u, 0u);
    __syncthreads();

    v16f acc[NB][MT];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int mi = 0; mi < MT; ++mi)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[nb][mi][i] = 0.f;
    // input staging: thread -> (row, sub-block of the stage's two); with fewer than 128 rows the upper threads idle
    const int tr = tid >> 1, tp = tid & 1;
    const bool a_thread = tr < kM;
    const int a_asg = a_thread ? s_asg[tr] : -1;
    const int64_t a_at = int64_t(max(a_asg, 0) / k.xdiv) * cols;
    // weights: lane (r, g) of wave w decodes sub-block g of the stage for weight row row0 + 32 w + r: its operand registers
    const int col = row0 + 32 * wave + r;
    const bool b_row = col < row_lim;
    const int64_t b_row_at = int64_t(e) * rows + (b_row ? col : row0);
    // loads run one stage ahead of their use; past the last sub-block they repeat it (the values are not used)
    RawX raw_a = load_x32(k.x, k.xtype, a_at + int64_t(min(tp, S - 1)) * 32);
    typename F16Sub<FMT>::Raw raw_b[NB];
#pragma unroll
    for (int bb = 0; bb < NB; ++bb) raw_b[bb] = F16Sub<FMT>::load(bb ? k.b1 : k.b0, b_row_at, min(g, S - 1));
    int buf = 0;
    for (int s0 = 0; s0 < s_end; s0 += 2, buf ^= 1) {
        // the loads of the next stage go out before this stage's conversions (a whole stage to arrive in) where the registers
        // allow a second set, else behind them
        constexpr bool kEarly = NB * MT < 8;
        RawX next_a;
        typename F16Sub<FMT>::Raw next_b[NB];
        if constexpr (kEarly) {
            next_a = load_x32(k.x, k.xtype, a_at + int64_t(min(s0 + 2 + tp, S - 1)) * 32);
#pragma unroll
            for (int bb = 0; bb < NB; ++bb) next_b[bb] = F16Sub<FMT>::load(bb ? k.b1 : k.b0, b_row_at, min(s0 + 2 + g, S - 1));
        }
        if (a_asg >= 0) {                       // rows without an assignment stay zero
            uint32_t h[16];
            finish_x32(raw_a, k.x, k.xtype, a_at + int64_t(min(s0 + tp, S - 1)) * 32, h);
            if (s0 + 2 > s_end) {               // the last stage of an odd number of sub-blocks (uniform)
                if (s0 + tp >= s_end) {
#pragma unroll
                    for (int i = 0; i < 16; ++i) h[i] = 0u;
                }
            }
#pragma unroll
            for (int q = 0; q < 4; ++q) *reinterpret_cast<uint4 *>(&As[buf][tr][tp * 32 + q * 8]) = make_uint4(h[4 * q], h[4 * q + 1], h[4 * q + 2], h[4 * q + 3]);
        }
        uint32_t hb[NB][16];
#pragma unroll
        for (int bb = 0; bb < NB; ++bb) {
            F16Sub<FMT>::finish(raw_b[bb], min(s0 + g, S - 1), grid, b_row && s0 + g < s_end, hb[bb]);
        }
        if constexpr (kEarly) {
            raw_a = next_a;
#pragma unroll
            for (int bb = 0; bb < NB; ++bb) raw_b[bb] = next_b[bb];
        } else {
            raw_a = load_x32(k.x, k.xtype, a_at + int64_t(min(s0 + 2 + tp, S - 1)) * 32);
#pragma unroll
            for (int bb = 0; bb < NB; ++bb) raw_b[bb] = F16Sub<FMT>::load(bb ? k.b1 : k.b0, b_row_at, min(s0 + 2 + g, S - 1));
        }
        // one barrier per stage: the tile written now was last read two stages ago, before the barrier of the stage between
        __syncthreads();
        // product j of a stage takes weights 8 j .. 8 j + 7 of the lane's sub-block; the input operand of lane (m, g) is the same
        // eight columns 32 g + 8 j .. of input row m (the order of the sum inside a stage is free as long as both agree)
        // all the block's tiles in straight-line code, also those without assignments (their input rows are zero): a branch per
        // tile would make every operand read wait by itself, and a second code path costs registers (and occupancy)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
#pragma unroll
            for (int m0 = 0; m0 < MT; m0 += 2) {   // two operand reads in flight, then their products
                constexpr int kPair = MT > 1 ? 2 : 1;
                v8h a[kPair];
#pragma unroll
                for (int mi = 0; mi < kPair; ++mi) a[mi] = *reinterpret_cast<const v8h *>(&As[buf][(m0 + mi) * 32 + r][32 * g + 8 * j]);
#pragma unroll
                for (int mi = 0; mi < kPair; ++mi)
#pragma unroll
                    for (int nb = 0; nb < NB; ++nb) {
                        const uint4 bw = make_uint4(hb[nb][4 * j], hb[nb][4 * j + 1], hb[nb][4 * j + 2], hb[nb][4 * j + 3]);
                        acc[nb][m0 + mi] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[mi], __builtin_bit_cast(v8h, bw), acc[nb][m0 + mi], 0, 0, 0);
                    }
                __builtin_amdgcn_sched_barrier(0);   // later reads stay behind these products (reading far ahead spills)
            }
        }
    }
    // result register i of lane half g: input row 8 (i / 4) + 4 g + i % 4 of the 32 x 32 tile, weight row r
    if (col >= rows) return;
#pragma unroll
    for (int mi = 0; mi < MT; ++mi)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int a = s_asg[mi * 32 + 8 * (i >> 2) + 4 * g + (i & 3)];
            if (a < 0) continue;
            float v = acc[0][mi][i];
            if (k.gateup) {
                float u = acc[NB - 1][mi][i];
                glu_clamp_inputs(k.glu, v, u);
                v = glu_clamp_silu(k.glu, v * __builtin_amdgcn_rcpf(1.f + __expf(-v))) * u;
            }
            v = col < row_lim ? v : 0.f;
            if (k.out_type == TQMOE_F32) static_cast<float *>(k.out)[int64_t(a) * rows + col] = v;
            else if (k.out_type == TQMOE_BF16) static_cast<uint16_t *>(k.out)[int64_t(a) * rows + col] = float_to_bf16_bits(v);
            else static_cast<uint16_t *>(k.out)[int64_t(a) * rows + col] = __half_as_ushort(__float2half_rn(v));
        }
}

}  // namespace

template <uint32_t FMT> void F16Launch<FMT>::run(const F16Args & k, bool two_banks, bool wide, dim3 grid, hipStream_t s) {
    if (wide) {
        if (two_banks) expert_gemm_f16_k<FMT, 2, 4><<<grid, 256, 0, s>>>(k); else expert_gemm_f16_k<FMT, 1, 4><<<grid, 256, 0, s>>>(k);
    } else {
        if (two_banks) expert_gemm_f16_k<FMT, 2, 2><<<grid, 256, 0, s>>>(k); else expert_gemm_f16_k<FMT, 1, 2><<<grid, 256, 0, s>>>(k);
    }
}

}  // namespace tqmoe

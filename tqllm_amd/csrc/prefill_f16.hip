// Prefill-sized expert products of any bank format: a grouped fp16 x fp16 -> fp32 GEMM on the matrix pipe.
//
// The counterpart of the reference's WeightFormat::expert_gemm / expert_gemm_gateup (weight_format.hpp:51-59): weights
// decoded to fp16 tiles in LDS, input rows converted to fp16, products accumulated in fp32 by
// v_mfma_f32_32x32x16_f16, gate and up in one launch with the SwiGLU epilogue. It serves the formats that have no int8
// grouped product of their own (Q4_K, IQ3_S, NVFP4G) and IQ4_XS shapes the int8 one does not take.
//
// A block takes one expert, up to 64 of its assignments (the dispatch lists give them) and 64 weight rows of each bank;
// its four waves hold one 32 x 32 quadrant each. Per 128 weights of a row (four sub-blocks) the block stages the
// 64 x 128 input tile and the 64 x 128 weight tile(s) in LDS (each weight row's sub-block decoded by one thread with the
// bank's exact decoder, then rounded to fp16) and every wave issues eight matrix instructions per bank.
#include "decode_api.cuh"
#include "decode_sub.cuh"

namespace tqmoe {
namespace {

typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int kRowsPerBlock = 64;   // assignments per block
constexpr int kKT = 128;            // weights of a row per stage
constexpr int kPad = kKT + 8;       // halves per staged row: 16-byte reads of consecutive rows spread over the LDS banks

struct F16Args {
    BankView b0, b1;
    uint32_t type;            // bank format
    const void * x;           // input rows of xtype, cols = bank cols
    const int * counts;       // [experts]
    const int * offsets;      // [experts + 1]
    const int * perm;         // assignment indices grouped by expert
    int experts;
    int xdiv;                 // input row of assignment a = a / xdiv
    void * out;               // [assignments][rows], fp16 or fp32
    int out_f32;
    int gateup;
    int shared_expert;        // the expert whose rows (gate / up) or columns (down) stop at shared_lim, or -1
    int shared_lim;
};

// the expert whose run of 64-row blocks holds `unit`; local = the block inside the expert; expert = -1 past the last
struct Where { int expert, local; };
__device__ __forceinline__ Where locate64(const int * __restrict__ counts, int experts, int unit) {
    __shared__ Where w;
    if (threadIdx.x < 64) {
        const int lane = threadIdx.x;
        if (lane == 0) w.expert = -1;
        int base = 0;
        for (int e0 = 0; e0 < experts; e0 += 64) {
            const int e = e0 + lane;
            const int units = e < experts ? (max(counts[e], 0) + kRowsPerBlock - 1) / kRowsPerBlock : 0;
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

__device__ __forceinline__ uint32_t pack_h2(float a, float b) {
    return uint32_t(__half_as_ushort(__float2half_rn(a))) | uint32_t(__half_as_ushort(__float2half_rn(b))) << 16;
}

template <int NB, int XT>
__global__ __launch_bounds__(256) void expert_gemm_f16_k(F16Args k) {
    __shared__ __attribute__((aligned(16))) uint16_t As[kRowsPerBlock][kPad];
    __shared__ __attribute__((aligned(16))) uint16_t Bs[NB][64][kPad];
    __shared__ int s_asg[kRowsPerBlock];
    const Where w = locate64(k.counts, k.experts, int(blockIdx.y));
    const int e = w.expert;
    if (e < 0) return;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, r = lane & 31, g = lane >> 5;
    const int mq = wave & 1, nq = wave >> 1;                   // quadrant: input rows 32 mq.., weight rows 32 nq.. of the block's 64 x 64
    const BankView & b0 = k.b0;
    const int rows = b0.rows, cols = b0.cols, S = cols / 32, row0 = int(blockIdx.x) * 64;
    const bool is_shared = e == k.shared_expert;
    const int row_lim = k.gateup && is_shared ? k.shared_lim : rows;     // weight rows this expert has
    const int s_end = !k.gateup && is_shared ? k.shared_lim / 32 : S;    // sub-blocks of the input rows it reads
    const int cnt = k.counts[e], first = w.local * kRowsPerBlock;
    if (tid < kRowsPerBlock) s_asg[tid] = first + tid < cnt ? k.perm[k.offsets[e] + first + tid] : -1;
    __syncthreads();

    v16f acc[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[nb][i] = 0.f;
    const int ar = tid >> 2, ap = tid & 3;                      // input staging: row, the sub-block of the stage's four
    const int a_asg = s_asg[ar];
    const int64_t a_at = int64_t(max(a_asg, 0) / k.xdiv) * cols + ap * 32;
    for (int s0 = 0; s0 < s_end; s0 += kKT / 32) {
        {
            uint4 h[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                float v[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
                if (a_asg >= 0) load8<XT>(k.x, a_at + int64_t(s0) * 32 + q * 8, v);
                h[q] = make_uint4(pack_h2(v[0], v[1]), pack_h2(v[2], v[3]), pack_h2(v[4], v[5]), pack_h2(v[6], v[7]));
            }
#pragma unroll
            for (int q = 0; q < 4; ++q) *reinterpret_cast<uint4 *>(&As[ar][ap * 32 + q * 8]) = h[q];
        }
        // weight staging: NB * 64 rows x 4 sub-blocks = NB * 256 decodes over the 256 threads
#pragma unroll
        for (int job = 0; job < NB; ++job) {
            const int idx = job * 256 + tid, bb = idx >> 8, bn = (idx >> 2) & 63, sub = idx & 3, s = s0 + sub;
            float y[32];
            if (row0 + bn < row_lim && s < s_end) {
                const BankView & b = bb ? k.b1 : k.b0;
                decode_sub32(k.type, b.codes, b.aux, b.rows_total, cols, int64_t(e) * rows + row0 + bn, s, y);
            } else {
#pragma unroll
                for (int i = 0; i < 32; ++i) y[i] = 0.f;
            }
#pragma unroll
            for (int q = 0; q < 4; ++q)
                *reinterpret_cast<uint4 *>(&Bs[bb][bn][sub * 32 + q * 8]) =
                    make_uint4(pack_h2(y[8 * q], y[8 * q + 1]), pack_h2(y[8 * q + 2], y[8 * q + 3]), pack_h2(y[8 * q + 4], y[8 * q + 5]), pack_h2(y[8 * q + 6], y[8 * q + 7]));
        }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < kKT / 16; ++j) {     // operand of lane (r, g): row r, columns 16 j + 8 g .. + 7
            const v8h a = *reinterpret_cast<const v8h *>(&As[mq * 32 + r][16 * j + 8 * g]);
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
                const v8h b = *reinterpret_cast<const v8h *>(&Bs[nb][nq * 32 + r][16 * j + 8 * g]);
                acc[nb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc[nb], 0, 0, 0);
            }
        }
        __syncthreads();
    }
    // result register i of lane half g: input row 8 (i / 4) + 4 g + i % 4 of the quadrant, weight row r
    const int col = row0 + nq * 32 + r;
    if (col >= rows) return;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const int a = s_asg[mq * 32 + 8 * (i >> 2) + 4 * g + (i & 3)];
        if (a < 0) continue;
        float v = acc[0][i];
        if (k.gateup) v = v / (1.f + expf(-v)) * acc[NB - 1][i];
        v = col < row_lim ? v : 0.f;
        if (k.out_f32) static_cast<float *>(k.out)[int64_t(a) * rows + col] = v;
        else static_cast<uint16_t *>(k.out)[int64_t(a) * rows + col] = __half_as_ushort(__float2half_rn(v));
    }
}

template <int NB>
void launch_f16(const F16Args & k, uint32_t xtype, dim3 grid, hipStream_t s) {
    switch (xtype) {
        case TQMOE_F32: expert_gemm_f16_k<NB, TQMOE_F32><<<grid, 256, 0, s>>>(k); break;
        case TQMOE_F16: expert_gemm_f16_k<NB, TQMOE_F16><<<grid, 256, 0, s>>>(k); break;
        default: expert_gemm_f16_k<NB, TQMOE_BF16><<<grid, 256, 0, s>>>(k); break;
    }
}

}  // namespace

// assignments = total entries of perm; the grid covers the most 64-row blocks the lists can need
int32_t enqueue_gemm_f16(const tqmoe_bank & b0, const tqmoe_bank * b1, const void * x, uint32_t xtype, const int * counts, const int * offsets, const int * perm,
                         int experts, int64_t assignments, int xdiv, void * out, int out_f32, int gateup, int shared_expert, int shared_lim, hipStream_t s) {
    const F16Args k{view(b0), b1 ? view(*b1) : view(b0), b0.type, x, counts, offsets, perm, experts, xdiv, out, out_f32, gateup, shared_expert, shared_lim};
    const int64_t units = assignments / kRowsPerBlock + experts;   // sum of ceil(count / 64) never exceeds this
    if (units > 65535) return -1;
    const dim3 grid(unsigned((b0.rows + 63) / 64), unsigned(units));
    if (b1) launch_f16<2>(k, xtype, grid, s); else launch_f16<1>(k, xtype, grid, s);
    return 0;
}

}  // namespace tqmoe

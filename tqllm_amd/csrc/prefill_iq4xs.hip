// Prefill-sized expert products of IQ4_XS banks: a grouped int8 x int8 -> int32 GEMM on the matrix pipe.
//
// Operands. Activations are int8 per input row (one fp32 scale per row, amax / 127), stored with every 32 values in the
// byte order of the bank's code bytes (see act_image.cuh: 16 bytes [16 g, 16 g + 16) hold values {8g..8g+7} and
// {16+8g..16+8g+7}). Weights are the bank's exact integer table values; the 6-bit sub-block scale is applied to the
// int32 result of each 32-wide product, the fp16 super-block scale once per 256, the row scale at the end. Nothing is
// rounded on the weight side.
//
// Blocks. The dispatch lists (counts, offsets, perm) give every expert's assignments. A block takes one expert, up to
// kMC of its assignments (32 per wave) and one tile of 32 weight rows. Per 256-weight super-block the block's four waves
// each decode two of the eight sub-blocks (v_perm_b32 lookups, 16 int8 values per lane) into an LDS tile that all waves
// then read as operand B of v_mfma_i32_32x32x32_i8, against operand A loaded straight from the activation rows. The tile
// is double-buffered: decoding super-block i + 1 overlaps the products of super-block i, one barrier per super-block.
#include "act_image.cuh"
#include "decode_api.cuh"
#include "formats.cuh"

namespace tqmoe {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kMC = 128;        // assignments per block
constexpr int kWaves = kMC / 32;

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

struct GemmArgs {
    BankView b0, b1;
    const int8_t * xq;        // [input rows][cols] int8, 32-blocks in bank byte order
    const float * xs;         // [input rows]
    const int * counts;       // [experts]
    const int * offsets;      // [experts + 1]
    const int * perm;         // assignment indices grouped by expert
    int experts;              // lists (bank matrices used)
    int xdiv;                 // input row of assignment a = a / xdiv
    uint16_t * out;           // fp16 [assignments][rows]: silu(gate) * up, or the plain product
    int gateup;
    int shared_expert;        // index of the expert whose rows (gate / up) or columns (down) stop at shared_lim, or -1
    int shared_lim;
};

// dynamic LDS: [2 buffers][NB][8 sub-blocks][64 lanes] v4i of decoded weights, then (experts + 1) ints for the chunk search
template <int NB>
__global__ __launch_bounds__(256) void iq4xs_gemm_k(GemmArgs k) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    v4i * bs = reinterpret_cast<v4i *>(lds);
    int * pre = reinterpret_cast<int *>(lds + 2 * NB * 8 * 64 * sizeof(v4i));
    __shared__ int s_expert, s_first, s_asg[kMC];
    __shared__ float s_scale[kMC];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, n = lane & 31, g = lane >> 5;

    // which expert and which kMC-chunk of its assignments: blockIdx.y counts chunks over the experts in order
    {
        const int E = k.experts;
        for (int e = tid; e < E; e += 256) pre[e] = (k.counts[e] + kMC - 1) / kMC;
        __syncthreads();
        if (wave == 0) {   // serial over 64-expert groups, ballot-free: a wave-wide inclusive scan per group
            int base = 0;
            for (int e0 = 0; e0 < E; e0 += 64) {
                const int e = e0 + lane;
                int v = e < E ? pre[e] : 0, incl = v;
#pragma unroll
                for (int d = 1; d < 64; d <<= 1) { const int t = __shfl_up(incl, d, 64); if (lane >= d) incl += t; }
                const int c = int(blockIdx.y);
                if (e < E && c >= base + incl - v && c < base + incl) { s_expert = e; s_first = (c - (base + incl - v)) * kMC; }
                base += __shfl(incl, 63, 64);
            }
            if (lane == 0 && int(blockIdx.y) >= base) s_expert = -1;
        }
        __syncthreads();
    }
    const int e = s_expert;
    if (e < 0) return;
    const BankView & b0 = k.b0;
    const int S = b0.cols / 32, NSB = S / 8, rows = b0.rows, tiles = rows / 32, tile = blockIdx.x;
    const bool is_shared = e == k.shared_expert;
    // gate / up rows of the shared expert beyond its size: no products, zeros stored (the rows are quantised whole later)
    const bool dead_tile = k.gateup && is_shared && tile * 32 >= k.shared_lim;
    const int sb_end = dead_tile ? 0 : !k.gateup && is_shared ? k.shared_lim / 256 : NSB;
    const int cnt = k.counts[e], first = s_first, here = min(kMC, cnt - first);
    if (tid < kMC) {
        const int a = tid < here ? k.perm[k.offsets[e] + first + tid] : -1;
        s_asg[tid] = a;
        s_scale[tid] = a >= 0 ? k.xs[a / k.xdiv] : 0.f;
    }
    __syncthreads();

    // operand A of this lane: row (32 wave + n) of the chunk, bytes [16 g, 16 g + 16) of every 32-block
    const int my_a = s_asg[32 * wave + n];
    const int8_t * a_ptr = k.xq + int64_t(max(my_a, 0) / k.xdiv) * b0.cols + g * 16;
    const bool wave_live = 32 * wave < here;
    const int64_t tile_g = int64_t(e) * tiles + tile;

    int acc_i[NB][16];
    float acc_f[NB][16];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int i = 0; i < 16; ++i) { acc_i[nb][i] = 0; acc_f[nb][i] = 0.f; }

    // this wave decodes sub-blocks 2 wave and 2 wave + 1 of every super-block, for each bank
    auto decode_into = [&](int sb, int buf) {
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
            const uint8_t * cp = (nb ? k.b1 : k.b0).codes + ((tile_g * S + int64_t(sb) * 8 + 2 * wave) * 32 + n) * 16 + g * 8;
#pragma unroll
            for (int j = 0; j < 2; ++j)
                bs[((buf * NB + nb) * 8 + 2 * wave + j) * 64 + lane] = decode16(*reinterpret_cast<const uint2 *>(cp + j * 512));
        }
    };
    decode_into(0, 0);
    __syncthreads();
    for (int sb = 0; sb < sb_end; ++sb) {
        const int buf = sb & 1;
        if (sb + 1 < sb_end) decode_into(sb + 1, buf ^ 1);
        if (wave_live) {
            uint2 rec[NB];
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) rec[nb] = *reinterpret_cast<const uint2 *>((nb ? k.b1 : k.b0).aux + ((tile_g * NSB + sb) * 32 + n) * 8);
            v4i areg[8];
#pragma unroll
            for (int ib = 0; ib < 8; ++ib) areg[ib] = my_a >= 0 ? *reinterpret_cast<const v4i *>(a_ptr + (sb * 8 + ib) * 32) : v4i{0, 0, 0, 0};
#pragma unroll
            for (int ib = 0; ib < 8; ++ib) {
#pragma unroll
                for (int nb = 0; nb < NB; ++nb) {
                    const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
                    const v16i d = __builtin_amdgcn_mfma_i32_32x32x32_i8(areg[ib], bs[((buf * NB + nb) * 8 + ib) * 64 + lane], zero, 0, 0, 0);
                    const int ls = iq4xs_ls(rec[nb], ib) - 32;
#pragma unroll
                    for (int i = 0; i < 16; ++i) acc_i[nb][i] += __mul24(d[i], ls);   // |d| < 2^19, |ls| <= 32: exact in 24-bit multiplies
                }
            }
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
                const float dsc = half_bits_to_float(uint16_t(rec[nb].x & 0xFFFFu));
#pragma unroll
                for (int i = 0; i < 16; ++i) { acc_f[nb][i] += float(acc_i[nb][i]) * dsc; acc_i[nb][i] = 0; }
            }
        }
        __syncthreads();
    }
    if (!wave_live) return;
    // result register i of lane half g is chunk row 32 wave + 8 (i / 4) + 4 g + i % 4, weight row n
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const int m = 32 * wave + 8 * (i >> 2) + 4 * g + (i & 3);
        const int a = s_asg[m];
        if (a < 0) continue;
        const float sc = s_scale[m];
        float v = acc_f[0][i] * sc;
        if (k.gateup) { const float u = acc_f[NB - 1][i] * sc; v = v / (1.f + expf(-v)) * u; }
        k.out[int64_t(a) * rows + tile * 32 + n] = __half_as_ushort(__float2half_rn(v));
    }
}

}  // namespace

// ---------------------------------------------------------------------------------------------- entry helpers
size_t prefill_lds_bytes(int nb, int experts) { return size_t(2) * nb * 8 * 64 * sizeof(v4i) + size_t(experts + 1) * sizeof(int); }

int32_t enqueue_quant_rows_i8(const void * x, uint32_t xtype, int64_t rows, int cols, int8_t * q, float * scale, hipStream_t s) {
    const unsigned blocks = unsigned((rows + 3) / 4);
    switch (xtype) {
        case TQMOE_F32: quant_rows_i8_k<TQMOE_F32><<<blocks, 256, 0, s>>>(x, rows, cols, q, scale); break;
        case TQMOE_F16: quant_rows_i8_k<TQMOE_F16><<<blocks, 256, 0, s>>>(x, rows, cols, q, scale); break;
        default: quant_rows_i8_k<TQMOE_BF16><<<blocks, 256, 0, s>>>(x, rows, cols, q, scale); break;
    }
    return 0;
}

// assignments = total entries of perm; the grid covers the most chunks the lists can need
int32_t enqueue_iq4xs_gemm(int nb, const tqmoe_bank & b0, const tqmoe_bank * b1, const int8_t * xq, const float * xs, const int * counts, const int * offsets,
                           const int * perm, int experts, int64_t assignments, int xdiv, void * out_f16, int gateup, int shared_expert, int shared_lim,
                           hipStream_t s) {
    GemmArgs k{view(b0), b1 ? view(*b1) : view(b0), xq, xs, counts, offsets, perm, experts, xdiv, static_cast<uint16_t *>(out_f16), gateup, shared_expert, shared_lim};
    const int64_t chunks = assignments / kMC + experts;   // sum of ceil(count / kMC) never exceeds this
    if (chunks > 65535) return -1;
    const dim3 grid(unsigned(b0.rows / 32), unsigned(chunks));
    const size_t lds = prefill_lds_bytes(nb, experts);
    if (nb == 2) iq4xs_gemm_k<2><<<grid, 256, lds, s>>>(k);
    else iq4xs_gemm_k<1><<<grid, 256, lds, s>>>(k);
    return 0;
}

}  // namespace tqmoe

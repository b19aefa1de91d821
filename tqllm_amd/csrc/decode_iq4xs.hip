// Decode-sized products of IQ4_XS banks on the matrix pipe.
//
// A block owns one expert, up to kTP of the input rows routed to it, and `tpw` tiles of 32 weight rows. Each wave takes
// one row tile and a share of the row's 256-weight super-blocks. Per 32-weight sub-block a lane (n = lane % 32,
// g = lane / 32) turns 8 code bytes of weight row n into 16 int8 table values with v_perm_b32 lookups; that is operand
// B of v_mfma_i32_32x32x32_i8. Operand A is the activation image: MFMA row 2j is the hi plane and row 2j + 1 the lo
// plane of input row j (rows past 2 kTP are zero), read straight from the image because its plane order is the order B's
// bytes come in. The MFMA does the 32-term sums for all rows and planes at once, so no lane exchange is needed; its
// result registers 0..3 of lane half g are (hi, lo) of input rows 2g and 2g + 1, which one fp32 multiply-add each folds
// into the lane's running sum with weight scale * activation scale. Waves that split a row's super-blocks add their
// partial sums through LDS in wave order (deterministic).
#include "act_image.cuh"
#include "decode_api.cuh"
#include "formats.cuh"

namespace tqmoe {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kTP = 4;         // input rows per block
constexpr int kMaxList = 2048; // assignments one block can scan (the launcher never passes more in mode 1)
constexpr int kMaxWaves = 8;

// The input rows this block serves. mode 0: its own assignment only. mode 1: the assignments of ids[0..A) with this
// block's expert, in index order, are cut into chunks of kTP; the block of each chunk's first assignment serves the
// chunk (returns its size and the assignment indices in tok, -1 past the end) and the other blocks leave (returns 0).
__device__ __forceinline__ int chunk_up(const int * __restrict__ ids, int A, int a, int e, int mode, int * list, int * meta, int (&tok)[kTP]) {
#pragma unroll
    for (int j = 0; j < kTP; ++j) tok[j] = -1;
    if (mode == 0) { tok[0] = a; return 1; }
    if (threadIdx.x < 64) {   // one wave walks the ids in order: ballots keep the matches ordered
        const int lane = threadIdx.x;
        int base = 0;
        for (int i0 = 0; i0 < A; i0 += 64) {
            const int i = i0 + lane;
            const bool match = i < A && ids[i] == e;
            const unsigned long long mask = __ballot(match);
            if (match) {
                const int r = base + __popcll(mask & ((1ull << lane) - 1ull));
                if (r < kMaxList) list[r] = i;
                if (i == a) meta[1] = r;
            }
            base += __popcll(mask);
        }
        if (lane == 0) meta[0] = min(base, kMaxList);
    }
    __syncthreads();
    const int cnt = meta[0], rank = meta[1];
    if (rank % kTP) return 0;
    const int n = min(kTP, cnt - rank);
#pragma unroll
    for (int j = 0; j < kTP; ++j) if (j < n) tok[j] = list[rank + j];
    return n;
}

// NB banks (gate and up, or one). gateup != 0: out0 is the activation image that receives silu(gate) * up; else out0 /
// out1 receive the products as rows of `ytype`. wk waves share a row's super-blocks, tpw row tiles per block.
template <int NB>
__global__ __launch_bounds__(512) void iq4xs_mfma_k(BankView b0, BankView b1, const uint8_t * __restrict__ image, void * out0, void * out1, uint32_t ytype,
                                                    const int * __restrict__ ids, int A, int xdiv, int mode, int slots, int topk, int shared_lim, int wk,
                                                    int tpw, int gateup) {
    __shared__ int list[kMaxList];
    __shared__ int meta[2], s_tok[kTP];
    __shared__ float red[kMaxWaves][NB][kTP][32];
    __shared__ int ql[kMaxWaves * 2][32];
    const int a = blockIdx.y, e = ids[a];
    if (e < 0 || int64_t(e) * b0.rows >= b0.rows_total) return;   // skipped assignment, or an id outside the bank
    int tok[kTP];
    const int n_tok = chunk_up(ids, A, a, e, mode, list, meta, tok);
    if (n_tok == 0) return;
    if (threadIdx.x < kTP) s_tok[threadIdx.x] = tok[threadIdx.x];
    __syncthreads();

    const int S = b0.cols / 32, NSB = S / 8, rows = b0.rows, tiles = rows / 32;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, n = lane & 31, g = lane >> 5;
    const int wk_i = wave % wk, rt_l = wave / wk, tile = blockIdx.x * tpw + rt_l;
    const bool shared_slot = (a % slots) >= topk;
    // the shared expert may have fewer rows (gate / up) or read a narrower input row (down)
    const int row_lim = gateup && shared_slot ? shared_lim : rows;
    const int s_end = !gateup && shared_slot ? shared_lim / 32 : S;
    const bool valid = tile < tiles && tile * 32 < row_lim;

    float accf[NB][2];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) accf[nb][0] = accf[nb][1] = 0.f;

    if (valid) {
        // this lane's part of operand A: plane row n of the MFMA = plane (n & 1) of input row n >> 1
        const int a_tok = n < 2 * kTP ? s_tok[n >> 1] : -1;
        const uint8_t * a_row = a_tok >= 0 ? image_row_ptr(image, a_tok / xdiv, S) + (n & 1) * 32 + g * 16 : nullptr;
        // the two input rows whose sums land in this lane half's result registers
        const int t0 = s_tok[2 * g], t1 = s_tok[2 * g + 1];
        const float * sc0 = t0 >= 0 ? image_scales(image_row_ptr(image, t0 / xdiv, S), S) : nullptr;
        const float * sc1 = t1 >= 0 ? image_scales(image_row_ptr(image, t1 / xdiv, S), S) : nullptr;
        const int64_t tile_g = int64_t(e) * tiles + tile;
        for (int sb = wk_i; sb < NSB; sb += wk) {
            v4i areg[8];
            float xs0[8], xs1[8];
#pragma unroll
            for (int ib = 0; ib < 8; ++ib) {
                const int s = sb * 8 + ib;
                const bool in = s < s_end;
                areg[ib] = a_row && in ? *reinterpret_cast<const v4i *>(a_row + int64_t(s) * 64) : v4i{0, 0, 0, 0};
                xs0[ib] = sc0 && in ? sc0[s] : 0.f;
                xs1[ib] = sc1 && in ? sc1[s] : 0.f;
            }
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
                const BankView & b = nb ? b1 : b0;
                const uint2 rec = *reinterpret_cast<const uint2 *>(b.aux + ((tile_g * NSB + sb) * 32 + n) * 8);
                const float d = half_bits_to_float(uint16_t(rec.x & 0xFFFFu));
                const uint8_t * cp = b.codes + ((tile_g * S + int64_t(sb) * 8) * 32 + n) * 16 + g * 8;
                uint2 c[8];
#pragma unroll
                for (int ib = 0; ib < 8; ++ib) c[ib] = *reinterpret_cast<const uint2 *>(cp + ib * 512);
#pragma unroll
                for (int ib = 0; ib < 8; ++ib) {
                    v4i bw;
                    uint32_t lo, hi;
                    lookup16<kIq4T0, kIq4T1, kIq4T2, kIq4T3>(c[ib].x, lo, hi);
                    bw[0] = int(lo); bw[1] = int(hi);
                    lookup16<kIq4T0, kIq4T1, kIq4T2, kIq4T3>(c[ib].y, lo, hi);
                    bw[2] = int(lo); bw[3] = int(hi);
                    v16i acc = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
                    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(areg[ib], bw, acc, 0, 0, 0);
                    const float ws = d * float(iq4xs_ls(rec, ib) - 32);
                    accf[nb][0] += float((acc[0] << 7) + acc[1]) * (ws * xs0[ib]);
                    accf[nb][1] += float((acc[2] << 7) + acc[3]) * (ws * xs1[ib]);
                }
            }
        }
    }
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) { red[wave][nb][2 * g][n] = accf[nb][0]; red[wave][nb][2 * g + 1][n] = accf[nb][1]; }
    __syncthreads();

    // the waves of a row tile hold the partial sums of its super-block shares: added here in wave order
    const int groups = tpw * kTP, per_pass = blockDim.x >> 5;
    for (int g0 = 0; g0 < groups; g0 += per_pass) {   // every wave runs every pass: the image quantiser exchanges lanes
        const int grp = g0 + (threadIdx.x >> 5), i = threadIdx.x & 31;
        const int rt = grp / kTP, j = grp % kTP, t = blockIdx.x * tpw + rt;
        const bool live = grp < groups && j < n_tok && t < tiles && t * 32 < row_lim;
        float v0 = 0.f, v1 = 0.f;
        if (live)
            for (int w = 0; w < wk; ++w) { v0 += red[rt * wk + w][0][j][i]; if (NB == 2) v1 += red[rt * wk + w][NB - 1][j][i]; }
        const int aj = live ? s_tok[j] : 0;
        if (gateup) {
            const float act = v0 / (1.f + expf(-v0)) * v1;
            quantise_block_lanes(act, i, live, ql[threadIdx.x >> 5], static_cast<uint8_t *>(out0) + int64_t(aj) * tiles * kImageSubBytes, tiles, t);
        } else if (live) {
            const int64_t o = int64_t(aj) * rows + t * 32 + i;
            if (ytype == TQMOE_F32) { static_cast<float *>(out0)[o] = v0; if (NB == 2) static_cast<float *>(out1)[o] = v1; }
            else { static_cast<uint16_t *>(out0)[o] = float_to_bf16_bits(v0); if (NB == 2) static_cast<uint16_t *>(out1)[o] = float_to_bf16_bits(v1); }
        }
    }
}

void launch(int nb, BankView b0, BankView b1, const uint8_t * image, void * out0, void * out1, uint32_t ytype, const int * ids, int A, int xdiv, int mode,
            int slots, int topk, int shared_lim, int gateup, hipStream_t s) {
    const int NSB = b0.cols / 256, tiles = b0.rows / 32;
    int wk = 1;
    for (int w = 1; w <= kMaxWaves; ++w) if (NSB % w == 0) wk = w;      // waves that share a row's super-blocks
    int tpw = kMaxWaves / wk;                                             // row tiles per block
    if (tpw > tiles) tpw = tiles;
    const dim3 grid(unsigned((tiles + tpw - 1) / tpw), unsigned(A));
    const unsigned threads = unsigned(wk * tpw * 64);
    if (nb == 2) iq4xs_mfma_k<2><<<grid, threads, 0, s>>>(b0, b1, image, out0, out1, ytype, ids, A, xdiv, mode, slots, topk, shared_lim, wk, tpw, gateup);
    else iq4xs_mfma_k<1><<<grid, threads, 0, s>>>(b0, b1, image, out0, out1, ytype, ids, A, xdiv, mode, slots, topk, shared_lim, wk, tpw, gateup);
}

}  // namespace

template <> void DecodeLaunch<TQMOE_IQ4_XS>::matvec(Split, int nb, const MatvecArgs & k, hipStream_t s) {
    launch(nb, k.b0, k.b1, k.image, k.y0, k.y1, k.ytype, k.ids, k.A, k.xdiv, k.mode, k.slots, k.topk, k.shared_cols, 0, s);
}
template <> void DecodeLaunch<TQMOE_IQ4_XS>::gateup(Split, const GateupArgs & k, hipStream_t s) {
    launch(2, k.bg, k.bu, k.ximage, k.aimage, nullptr, TQMOE_F32, k.ids, k.A, k.slots, k.mode, k.slots, k.topk, k.shared_ff, 1, s);
}

}  // namespace tqmoe

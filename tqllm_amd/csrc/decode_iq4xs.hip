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
// The weight bytes are the only cold data: every wave loads its share (codes and scale records) into registers one
// super-block ahead of the one it is multiplying, so the loads of the next super-block are in flight while this one is
// decoded.
#include "act_image.cuh"
#include "decode_chunks.cuh"
#include "decode_api.cuh"
#include "formats.cuh"

namespace tqmoe {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kTP = kChunkRowsMax;   // input rows per block
constexpr int kMaxWaves = 8;

// 16 four-bit codes (two dwords) -> operand B of the MFMA: the lookups of lookup16(). The selector of the third pick
// is (bit 3 of the code at bit 2) | byte position: one v_and_or_b32 when the mask and the positions sit in registers
// (k4 in a vector register, pos in a scalar one; as literals the instruction cannot encode them and the compiler
// splits it in two).
struct NibbleConsts { uint32_t k4, pos; };
__device__ __forceinline__ NibbleConsts nibble_consts() {
    NibbleConsts c{0x04040404u, 0x03020100u};
    asm volatile("" : "+v"(c.k4));
    asm volatile("" : "+s"(c.pos));
    return c;
}
__device__ __forceinline__ v4i decode16(uint2 c, NibbleConsts nc) {
    v4i w;
    const uint32_t k7 = 0x07070707u;
    const uint32_t x0 = c.x, x1 = c.y;
    const uint32_t i0 = x0 & k7, j0 = (x0 >> 4) & k7, i1 = x1 & k7, j1 = (x1 >> 4) & k7;
    w[0] = int(__builtin_amdgcn_perm(__builtin_amdgcn_perm(kIq4T3, kIq4T2, i0), __builtin_amdgcn_perm(kIq4T1, kIq4T0, i0), ((x0 >> 1) & nc.k4) | nc.pos));
    w[1] = int(__builtin_amdgcn_perm(__builtin_amdgcn_perm(kIq4T3, kIq4T2, j0), __builtin_amdgcn_perm(kIq4T1, kIq4T0, j0), ((x0 >> 5) & nc.k4) | nc.pos));
    w[2] = int(__builtin_amdgcn_perm(__builtin_amdgcn_perm(kIq4T3, kIq4T2, i1), __builtin_amdgcn_perm(kIq4T1, kIq4T0, i1), ((x1 >> 1) & nc.k4) | nc.pos));
    w[3] = int(__builtin_amdgcn_perm(__builtin_amdgcn_perm(kIq4T3, kIq4T2, j1), __builtin_amdgcn_perm(kIq4T1, kIq4T0, j1), ((x1 >> 5) & nc.k4) | nc.pos));
    return w;
}

// NB banks (gate and up, or one). gateup != 0: out0 is the activation image that receives silu(gate) * up; else out0 /
// out1 receive the products as rows of `ytype`. wk waves share a row's super-blocks, tpw row tiles per block.
// Dynamic LDS: the match list and the copy of the ids while the block finds its input rows, later the partial sums.
// UNI: every sub-block of an input row has the row's one activation scale (the images tqmoe_quant_act and the top-k
// kernel write). The 6-bit weight scales then multiply the integer results and the sums stay integers over a whole
// super-block; otherwise (rows quantised block by block, as the fused gate / up epilogue leaves them) each sub-block's
// result is scaled in fp32.
// MODE 0: input rows read straight from the image; 1: staged in LDS; 2: staged, and a wave takes tl_count row tiles in turn
template <int NB, bool UNI, int MODE>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(3))) void iq4xs_mfma_k(BankView b0, BankView b1, const uint8_t * __restrict__ image, void * out0, void * out1, uint32_t ytype,
                                                    const int * __restrict__ ids, int A, int xdiv, int mode, int slots, int topk, int shared_lim, int wk,
                                                    int tpw, int gateup, int a_off, int tl_count, Glu glu) {
    constexpr bool STAGED = MODE >= 1, MULTI = MODE == 2;
    extern __shared__ __attribute__((aligned(16))) uint8_t stage[];
    __shared__ int meta[2], s_tok[kTP];
    __shared__ float s_x0[kTP];
    __shared__ int ql[kMaxWaves * 2][32];
    const int a = blockIdx.y, e = fetch_ids(ids, A, a, mode, reinterpret_cast<int *>(stage));
    if (e < 0 || int64_t(e) * b0.rows >= b0.rows_total) return;   // skipped assignment, or an id outside the bank
    int tok[kTP];
    const int n_tok = chunk_up(A, a, e, mode, kTP, reinterpret_cast<int *>(stage), meta, tok);   // the lists live in the dynamic space
    if (n_tok == 0) return;
    if (threadIdx.x < kTP) s_tok[threadIdx.x] = tok[threadIdx.x];

    const int S = b0.cols / 32, NSB = S / 8, rows = b0.rows, tiles = rows / 32;
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), n = lane & 31, g = lane >> 5;
    const int wk_i = wave % wk, rt_l = wave / wk, tile = blockIdx.x * tl_count * tpw + rt_l;   // the wave's first (or only) row tile
    const bool shared_slot = (a % slots) >= topk;
    // the shared expert may have fewer rows (gate / up) or read a narrower input row (down)
    const int row_lim = gateup && shared_slot ? shared_lim : rows;
    const int s_end = !gateup && shared_slot ? shared_lim / 32 : S;
    const bool valid = tile < tiles && tile * 32 < row_lim;

    // The weight bytes of a super-block: 8 bytes of codes per sub-block and the row's scale record, per lane, in
    // registers. The next super-block's are loaded before this one is multiplied (into the other of two sets that swap
    // roles, no copies), so that there are always loads in flight under the decode work. Past the wave's last
    // super-block the same one is fetched again: a branch around the loads would make every wait a wait for all of them.
    // The first super-block's loads go out before the input rows are staged: the two trips to memory overlap.
    const int sb_end = s_end / 8;   // whole super-blocks only (the launcher checks)
    const bool working = valid && wk_i < sb_end;
    struct Cold { uint2 code[NB][8]; uint2 rec[NB]; };
    // the lane's addresses in the wave's first row tile, worked out once; a fetch adds 32-bit offsets (dt row tiles further on)
    const uint8_t * code_base[NB], * rec_base[NB];
    {
        const int64_t tile_g = int64_t(e) * tiles + tile;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
            code_base[nb] = (nb ? b1 : b0).codes + tile_g * S * 512 + n * 16 + g * 8;
            rec_base[nb] = (nb ? b1 : b0).aux + tile_g * NSB * 256 + n * 8;
        }
    }
    auto fetch_tile = [&](int dt, int sb, Cold & c) {
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
            const uint8_t * src = code_base[nb] + uint32_t(dt * S + sb * 8) * 512u;
#pragma unroll
            for (int ib = 0; ib < 8; ++ib) c.code[nb][ib] = *reinterpret_cast<const uint2 *>(src + ib * 512);
            c.rec[nb] = *reinterpret_cast<const uint2 *>(rec_base[nb] + uint32_t(dt * NSB + sb) * 256u);
        }
    };
    auto fetch = [&](int sb, Cold & c) { fetch_tile(0, sb, c); };
    Cold c0, c1;
    if (working) fetch(wk_i, c0);
    // The planes and scales of the block's input rows go to LDS once: [sub-block][input row][64 bytes of planes], then
    // [input row][sub-block] scales. The product loop then has no loads from memory but the weights', so that its waits
    // count exactly those (a wait for an operand A load would also wait for every weight load issued before it).
    uint8_t * a_lds = stage + a_off;
    float * xs_lds = reinterpret_cast<float *>(a_lds + S * 256);
    if constexpr (STAGED) {
        const uint8_t * src_row[kTP];
#pragma unroll
        for (int j = 0; j < kTP; ++j) src_row[j] = image_row_ptr(image, (tok[j] >= 0 ? tok[j] : tok[0]) / xdiv, S);   // rows not served: the first row's
        for (int i0 = threadIdx.x; i0 < S * 16; i0 += 4 * blockDim.x) {   // four pieces a thread per trip to memory
            auto piece = [&](int q) {   // past the end: the last piece again, not stored
                const int i = min(i0 + q * int(blockDim.x), S * 16 - 1), j = (i >> 2) & 3;
                const uint8_t * row = j == 0 ? src_row[0] : j == 1 ? src_row[1] : j == 2 ? src_row[2] : src_row[3];
                return *reinterpret_cast<const uint4 *>(row + (i >> 4) * 64 + (i & 3) * 16);
            };
            auto put = [&](int q, const uint4 & v) {
                const int i = i0 + q * int(blockDim.x);
                if (i < S * 16) *reinterpret_cast<uint4 *>(a_lds + i * 16) = v;
            };
            // (four named values, not an array: an array indexed in two loops has been placed in scratch memory by the compiler,
            // one trip to memory per piece)
            const uint4 v0 = piece(0), v1 = piece(1), v2 = piece(2), v3 = piece(3);
            put(0, v0); put(1, v1); put(2, v2); put(3, v3);
        }
        if constexpr (UNI) {   // the rows' one scale each
            if (threadIdx.x < kTP) {
                const int j = threadIdx.x;
                s_x0[j] = image_scales(j == 0 ? src_row[0] : j == 1 ? src_row[1] : j == 2 ? src_row[2] : src_row[3], S)[0];
            }
        } else
            for (int i = threadIdx.x; i < S * kTP; i += blockDim.x) {
                const int j = i / S;
                const uint8_t * row = j == 0 ? src_row[0] : j == 1 ? src_row[1] : j == 2 ? src_row[2] : src_row[3];
                xs_lds[i] = image_scales(row, S)[i - j * S];
            }
    }
    __syncthreads();

    float accf[NB][2];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) accf[nb][0] = accf[nb][1] = 0.f;

    // A row tile's sums to their place. tile0: the block's first row tile of this pass.
    auto finish = [&](int tile0, bool wave_valid) {
        if constexpr (UNI) {
            if (wave_valid) {   // the rows' own scales, once
                const float x0 = STAGED ? s_x0[2 * g] : image_scales(image_row_ptr(image, max(s_tok[2 * g], 0) / xdiv, S), S)[0];
                const float x1 = STAGED ? s_x0[2 * g + 1] : image_scales(image_row_ptr(image, max(s_tok[2 * g + 1], 0) / xdiv, S), S)[0];
#pragma unroll
                for (int nb = 0; nb < NB; ++nb) { accf[nb][0] *= x0; accf[nb][1] *= x1; }
            }
        }
        __syncthreads();                                       // the id list (or the previous pass's sums) is done with: the space now holds the partial sums
        float (*red)[NB][kTP][32] = reinterpret_cast<float (*)[NB][kTP][32]>(stage);
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) { red[wave][nb][2 * g][n] = accf[nb][0]; red[wave][nb][2 * g + 1][n] = accf[nb][1]; }
        __syncthreads();

        // the waves of a row tile hold the partial sums of its super-block shares: added here in wave order
        const int groups = tpw * kTP, per_pass = blockDim.x >> 5;
        for (int g0 = 0; g0 < groups; g0 += per_pass) {   // every wave runs every pass: the image quantiser exchanges lanes
            const int grp = g0 + (threadIdx.x >> 5), i = threadIdx.x & 31;
            const int rt = grp / kTP, j = grp % kTP, t = tile0 + rt;
            const bool live = grp < groups && j < n_tok && t < tiles && t * 32 < row_lim;
            float v0 = 0.f, v1 = 0.f;
            if (live)
                for (int w = 0; w < wk; ++w) { v0 += red[rt * wk + w][0][j][i]; if (NB == 2) v1 += red[rt * wk + w][NB - 1][j][i]; }
            const int aj = live ? s_tok[j] : 0;
            if (gateup) {
                glu_clamp_inputs(glu, v0, v1);
                const float act = glu_clamp_silu(glu, v0 / (1.f + expf(-v0))) * v1;
                quantise_block_lanes(act, i, live, ql[threadIdx.x >> 5], static_cast<uint8_t *>(out0) + int64_t(aj) * tiles * kImageSubBytes, tiles, t);
            } else if (live) {
                const int64_t o = int64_t(aj) * rows + t * 32 + i;
                if (ytype == TQMOE_F32) { static_cast<float *>(out0)[o] = v0; if (NB == 2) static_cast<float *>(out1)[o] = v1; }
                else { static_cast<uint16_t *>(out0)[o] = float_to_bf16_bits(v0); if (NB == 2) static_cast<uint16_t *>(out1)[o] = float_to_bf16_bits(v1); }
            }
        }
    };

    if (working) {
        // this lane's part of operand A: plane row n of the MFMA = plane (n & 1) of input row n >> 1 (rows 8 and up repeat
        // rows 0..7: their sums land in result rows that nobody reads)
        // (not staged: straight from the image, a stride of 64 bytes per sub-block instead of the staged 256)
        const int a_tok = max(s_tok[(n & 7) >> 1], s_tok[0]);
        const uint8_t * a_lane = STAGED ? a_lds + ((n & 7) >> 1) * 64 + (n & 1) * 32 + g * 16 : image_row_ptr(image, a_tok / xdiv, S) + (n & 1) * 32 + g * 16;
        constexpr int kStrideA = STAGED ? 256 : 64;
        // the two input rows whose sums land in this lane half's result registers
        const float * sc0 = STAGED ? xs_lds + (2 * g) * S : image_scales(image_row_ptr(image, max(s_tok[2 * g], 0) / xdiv, S), S);
        const float * sc1 = STAGED ? xs_lds + (2 * g + 1) * S : image_scales(image_row_ptr(image, max(s_tok[2 * g + 1], 0) / xdiv, S), S);
        const NibbleConsts ncs = nibble_consts();
        auto multiply = [&](int sb, const Cold & cur) {
            v4i areg[8];
#pragma unroll
            for (int ib = 0; ib < 8; ++ib) areg[ib] = *reinterpret_cast<const v4i *>(a_lane + (sb * 8 + ib) * kStrideA);
            // activation scales of the 8 sub-blocks
            float xs0[8], xs1[8];
            if constexpr (!UNI) {
                const float4 p0 = *reinterpret_cast<const float4 *>(sc0 + sb * 8), p1 = *reinterpret_cast<const float4 *>(sc0 + sb * 8 + 4);
                const float4 q0 = *reinterpret_cast<const float4 *>(sc1 + sb * 8), q1 = *reinterpret_cast<const float4 *>(sc1 + sb * 8 + 4);
                xs0[0] = p0.x; xs0[1] = p0.y; xs0[2] = p0.z; xs0[3] = p0.w; xs0[4] = p1.x; xs0[5] = p1.y; xs0[6] = p1.z; xs0[7] = p1.w;
                xs1[0] = q0.x; xs1[1] = q0.y; xs1[2] = q0.z; xs1[3] = q0.w; xs1[4] = q1.x; xs1[5] = q1.y; xs1[6] = q1.z; xs1[7] = q1.w;
            }
            // The products of step (bank, sub-block) + 1 are issued before the sums of this step are read: the matrix pipe's
            // latency passes under the next step's lookups instead of in front of this step's multiply-adds.
            const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
            // steps in the order (sub-block, bank): a sub-block's piece of operand A serves the banks one after the other
            auto issue = [&](int step) {
                return __builtin_amdgcn_mfma_i32_32x32x32_i8(areg[step / NB], decode16(cur.code[step % NB][step / NB], ncs), zero, 0, 0, 0);
            };
            constexpr bool kAhead = UNI;   // the other kernels lose more to the registers of a second result than they gain
            v16i acc = issue(0);
            int si[NB][4];   // (hi, lo) plane sums of the two input rows, weighted by the sub-block scales
#pragma unroll
            for (int step = 0; step < 8 * NB; ++step) {
                const int nb = step % NB, ib = step / NB;
                v16i ahead = zero;
                if constexpr (kAhead) {
                    if (step + 1 < 8 * NB) ahead = issue(step + 1);
                    __builtin_amdgcn_sched_barrier(0);
                }
                const uint2 rec = cur.rec[nb];
                if constexpr (UNI) {
                    // |acc| <= 32 * 128 * 127 < 2^19 and |ls - 32| <= 32: 24-bit products, eight of them stay below 2^28
                    const int ls = iq4xs_lsm32(rec, ib);
#pragma unroll
                    for (int q = 0; q < 4; ++q) si[nb][q] = (ib ? si[nb][q] : 0) + __mul24(acc[q], ls);
                    if (ib == 7) {
                        const float d = half_bits_to_float(iq4xs_d_bits(rec));
                        accf[nb][0] += (float(si[nb][0]) * 128.f + float(si[nb][1])) * d;
                        accf[nb][1] += (float(si[nb][2]) * 128.f + float(si[nb][3])) * d;
                    }
                } else {
                    const float ws = half_bits_to_float(iq4xs_d_bits(rec)) * float(iq4xs_lsm32(rec, ib));
                    accf[nb][0] += float((acc[0] << 7) + acc[1]) * (ws * xs0[ib]);
                    accf[nb][1] += float((acc[2] << 7) + acc[3]) * (ws * xs1[ib]);
                }
                // only four of the sixteen result registers are read; the others count as in use until here, or they are handed
                // to the next lookups while the matrix pipe still writes them and every such write waits for the pipe
                asm volatile("" : : "v"(acc));
                if constexpr (kAhead) acc = ahead;
                else if (step + 1 < 8 * NB) acc = issue(step + 1);
            }
        };
        if constexpr (MULTI) {
            // Several row tiles a wave, one after the other (the launcher has made sure that every wave of the block has the
            // same steps: no ragged tiles, no shorter shared expert): the block finds its input rows and stages them once, and
            // the weight loads run on across the tiles' ends, the next tile's first under this tile's sums.
            const int nsteps = sb_end / wk, total = tl_count * nsteps;
            auto fetch_step = [&](int gs, Cold & c) { fetch_tile(gs / nsteps * tpw, wk_i + gs % nsteps * wk, c); };
            auto after = [&](int gs) {   // step gs is done: was it its tile's last?
                if ((gs + 1) % nsteps) return;
                finish((int(blockIdx.x) * tl_count + gs / nsteps) * tpw, true);
#pragma unroll
                for (int nb = 0; nb < NB; ++nb) accf[nb][0] = accf[nb][1] = 0.f;
            };
            for (int gs = 0; gs < total; gs += 2) {
                fetch_step(min(gs + 1, total - 1), c1);
                multiply(wk_i + gs % nsteps * wk, c0);
                after(gs);
                if (gs + 1 >= total) break;
                fetch_step(min(gs + 2, total - 1), c0);
                multiply(wk_i + (gs + 1) % nsteps * wk, c1);
                after(gs + 1);
            }
        } else if constexpr (STAGED) {
            const int last = wk_i + (sb_end - 1 - wk_i) / wk * wk;   // the wave's last super-block
            for (int sb = wk_i; sb <= last; sb += 2 * wk) {
                fetch(min(sb + wk, last), c1);
                multiply(sb, c0);
                if (sb + wk > last) break;
                fetch(min(sb + 2 * wk, last), c0);
                multiply(sb + wk, c1);
            }
        } else {   // short batches: most waves have one super-block, and nothing is fetched that is not multiplied
            for (int sb = wk_i; sb < sb_end; sb += wk) {
                if (sb + wk < sb_end) fetch(sb + wk, c1);
                multiply(sb, c0);
                c0 = c1;
            }
        }
    }

    if constexpr (!MULTI) finish(blockIdx.x * tpw, valid);
}

void launch(int nb, BankView b0, BankView b1, const uint8_t * image, void * out0, void * out1, uint32_t ytype, const int * ids, int A, int xdiv, int mode,
            int slots, int topk, int shared_lim, int gateup, bool uniform, Glu glu, hipStream_t s) {
    const int NSB = b0.cols / 256, tiles = b0.rows / 32;
    // Waves that share a row's super-blocks: as many as it takes to put a few thousand waves in flight (a short batch
    // is bound by the latency of one wave's chain), fewer when the batch has the waves anyway (a longer chain per
    // wave streams with its loads one super-block ahead and saves the cross-wave sums).
    const int64_t units = int64_t(A) * tiles;
    const int cap = units >= 8192 ? 1 : units >= 2048 ? 2 : units >= 512 ? 4 : kMaxWaves;
    int wk = 1;
    for (int w = 1; w <= kMaxWaves && w <= cap; ++w) if (NSB % w == 0) wk = w;
    const int waves = wk == kMaxWaves ? kMaxWaves : 4;                    // per block: small blocks, a compute unit holds several and their phases interleave
    int tpw = waves / wk;                                                 // row tiles per block
    if (tpw > tiles) tpw = tiles;
    const unsigned threads = unsigned(wk * tpw * 64);
    // dynamic LDS: the match list and the copy of the ids (2 * kMaxList ints), later the partial sums; behind them the input
    // rows' planes (256 bytes per sub-block) and, for rows with a scale per sub-block, the scales
    size_t lds = mode ? size_t(2) * kMaxList * sizeof(int) : 0;
    if (lds < size_t(wk * tpw) * nb * kTP * 32 * sizeof(float)) lds = size_t(wk * tpw) * nb * kTP * 32 * sizeof(float);
    // the input rows go through LDS from a dozen tokens on (measured: 5 % at 16 and 32 tokens; the waves then overlap each
    // other's waits, and what counts is that a wave's own weight loads stay in flight under its products); a short batch is
    // one chain of dependent steps per wave, and the extra stop at a barrier costs more than the exact waits return
    const bool staged = A >= 12 * slots;
    // ... and a wave then takes up to four row tiles one after the other, as long as the grid keeps two blocks per compute
    // unit: the block's search for its input rows and their staging are paid once for all of them
    int tl = 1;
    if (staged && nb == 1 && shared_lim == (gateup ? b0.rows : b0.cols))
        while (tl < 4 && tiles % (tpw * tl * 2) == 0 && int64_t(tiles / (tpw * tl * 2)) * A >= 512) tl *= 2;
    const dim3 grid(unsigned((tiles + tpw * tl - 1) / (tpw * tl)), unsigned(A));
    const int a_off = int(lds);
    if (staged) lds += size_t(b0.cols / 32) * (256 + (uniform ? 0 : kTP * sizeof(float)));
    auto go = [&](auto kernel) { kernel<<<grid, threads, lds, s>>>(b0, b1, image, out0, out1, ytype, ids, A, xdiv, mode, slots, topk, shared_lim, wk, tpw, gateup, a_off, tl, glu); };
    if (nb == 2 && uniform) staged ? go(iq4xs_mfma_k<2, true, 1>) : go(iq4xs_mfma_k<2, true, 0>);
    else if (nb == 2) staged ? go(iq4xs_mfma_k<2, false, 1>) : go(iq4xs_mfma_k<2, false, 0>);
    else if (tl > 1) go(iq4xs_mfma_k<1, false, 2>);
    else staged ? go(iq4xs_mfma_k<1, false, 1>) : go(iq4xs_mfma_k<1, false, 0>);
}

}  // namespace

template <> void DecodeLaunch<TQMOE_IQ4_XS>::matvec(Split, int nb, const MatvecArgs & k, hipStream_t s) {
    launch(nb, k.b0, k.b1, k.image, k.y0, k.y1, k.ytype, k.ids, k.A, k.xdiv, k.mode, k.slots, k.topk, k.shared_cols, 0, false, Glu{0.f, 0}, s);
}
template <> void DecodeLaunch<TQMOE_IQ4_XS>::gateup(Split, const GateupArgs & k, hipStream_t s) {
    launch(2, k.bg, k.bu, k.ximage, k.aimage, nullptr, TQMOE_F32, k.ids, k.A, k.slots, k.mode, k.slots, k.topk, k.shared_ff, 1, true, k.glu, s);
}

}  // namespace tqmoe

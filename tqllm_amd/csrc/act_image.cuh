// The activation image the decode products read (layout: include/tqmoe.h) and its quantiser.
//
// One image row of `cols` values, S = cols / 32 sub-blocks:
//   [S][64 B]  per sub-block the hi plane (32 int8) then the lo plane (32 int8), q = 128 * hi + lo, q = rint(x / scale);
//              inside a plane the eight dwords are stored in the order 0, 4, 1, 5, 2, 6, 3, 7 of the natural dwords
//              (natural dword d = values 4d .. 4d + 3), so that the 16 bytes [16 g, 16 g + 16) are exactly the values
//              {8g .. 8g + 7} and {16 + 8g .. 16 + 8g + 7}: the two halves of a sub-block that pair with code bytes
//              8g .. 8g + 7 of a 4-bit bank (low nibbles = values 0..15, high nibbles = values 16..31);
//   [S] fp32   scale of each sub-block: amax / 16383 of the block, or of the whole row (every entry the same) for the
//              rows quantise_row_wave writes;
//   [S] fp32   sum of the sub-block's q times its scale (the term a per-block minimum multiplies).
#pragma once
#include "common.cuh"

namespace tqmoe {
namespace {

constexpr int kImageSubBytes = 72;  // bytes of an image row per sub-block: 64 of planes, 4 of scale, 4 of sum

// plane position of natural dword d (0..7)
__host__ __device__ constexpr int plane_pos(int d) { return d < 4 ? 2 * d : 2 * (d - 4) + 1; }

struct ActBlock { int hi[8], lo[8]; float scale, sum; };   // hi / lo indexed by plane position

__device__ __forceinline__ const uint8_t * image_row_ptr(const uint8_t * image, int64_t row, int S) { return image + row * S * kImageSubBytes; }
__device__ __forceinline__ const float * image_scales(const uint8_t * image_row, int S) { return reinterpret_cast<const float *>(image_row + int64_t(S) * 64); }
__device__ __forceinline__ const float * image_sums(const uint8_t * image_row, int S) { return reinterpret_cast<const float *>(image_row + int64_t(S) * 68); }

__device__ __forceinline__ void load_act_block(const uint8_t * __restrict__ image_row, int S, int s, ActBlock & b) {
    const uint4 * p = reinterpret_cast<const uint4 *>(image_row + int64_t(s) * 64);
    const uint4 a0 = p[0], a1 = p[1], a2 = p[2], a3 = p[3];
    b.hi[0] = a0.x; b.hi[1] = a0.y; b.hi[2] = a0.z; b.hi[3] = a0.w; b.hi[4] = a1.x; b.hi[5] = a1.y; b.hi[6] = a1.z; b.hi[7] = a1.w;
    b.lo[0] = a2.x; b.lo[1] = a2.y; b.lo[2] = a2.z; b.lo[3] = a2.w; b.lo[4] = a3.x; b.lo[5] = a3.y; b.lo[6] = a3.z; b.lo[7] = a3.w;
    b.scale = image_scales(image_row, S)[s];
    b.sum = image_sums(image_row, S)[s];
}
__device__ __forceinline__ void zero_act_block(ActBlock & b) {
#pragma unroll
    for (int i = 0; i < 8; ++i) { b.hi[i] = 0; b.lo[i] = 0; }
    b.scale = 0.f;
    b.sum = 0.f;
}

__device__ __forceinline__ float block_amax(const float (&v)[32]) {
    float amax = 0.f;
#pragma unroll
    for (int i = 0; i < 32; ++i) amax = fmaxf(amax, fabsf(v[i]));
    return amax;
}

// 32 values (natural order) -> sub-block s of an image row, quantised against `amax` (the block's own maximum, or the
// maximum of a larger set that contains the block: the whole row for the rows tqmoe_quant_act writes)
__device__ __forceinline__ void quantise_block(const float (&v)[32], uint8_t * image_row, int S, int s, float amax) {
    const float scale = amax * (1.f / 16383.f), inv = amax > 0.f ? 16383.f / amax : 0.f;
    uint32_t hi[8], lo[8];
    int qsum = 0;
#pragma unroll
    for (int d = 0; d < 8; ++d) {
        uint32_t h = 0, l = 0;
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            const int q = __float2int_rn(v[4 * d + b] * inv);
            qsum += q;
            h |= uint32_t((q >> 7) & 0xFF) << (8 * b);
            l |= uint32_t(q & 127) << (8 * b);
        }
        hi[plane_pos(d)] = h;
        lo[plane_pos(d)] = l;
    }
    uint4 * p = reinterpret_cast<uint4 *>(image_row + int64_t(s) * 64);
    p[0] = make_uint4(hi[0], hi[1], hi[2], hi[3]);
    p[1] = make_uint4(hi[4], hi[5], hi[6], hi[7]);
    p[2] = make_uint4(lo[0], lo[1], lo[2], lo[3]);
    p[3] = make_uint4(lo[4], lo[5], lo[6], lo[7]);
    reinterpret_cast<float *>(image_row + int64_t(S) * 64)[s] = scale;
    reinterpret_cast<float *>(image_row + int64_t(S) * 68)[s] = float(qsum) * scale;
}

// 32 values held one per lane by 32 consecutive lanes (lane i of the group has value i; every lane of the wave must
// call this) -> sub-block s of an image row. q_lds: 32 ints of LDS private to the group. live: whether to store.
__device__ __forceinline__ void quantise_block_lanes(float v, int i, bool live, int * q_lds, uint8_t * image_row, int S, int s) {
    float amax = fabsf(v);
    amax = fmaxf(amax, dpp_f<kDppXor1>(amax));
    amax = fmaxf(amax, dpp_f<kDppXor2>(amax));
    amax = fmaxf(amax, dpp_f<kDppHalfMirror>(amax));
    amax = fmaxf(amax, dpp_f<kDppMirror>(amax));
    amax = fmaxf(amax, __shfl_xor(amax, 16, 64));
    const float inv = amax > 0.f ? 16383.f / amax : 0.f;
    const int q = __float2int_rn(v * inv);
    q_lds[i] = q;
    int qs = q;
    qs += dpp_i<kDppXor1>(qs);
    qs += dpp_i<kDppXor2>(qs);
    qs += dpp_i<kDppHalfMirror>(qs);
    qs += dpp_i<kDppMirror>(qs);
    qs += __shfl_xor(qs, 16, 64);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");   // q_lds is read below by other lanes of this same wave
    __builtin_amdgcn_wave_barrier();
    if (!live) return;
    if (i < 16) {   // lanes 0..7 build the hi plane's dwords, 8..15 the lo plane's
        const int d = i & 7;
        uint32_t word = 0;
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            const int qq = q_lds[4 * d + b];
            word |= uint32_t(i < 8 ? (qq >> 7) & 0xFF : qq & 127) << (8 * b);
        }
        reinterpret_cast<uint32_t *>(image_row + int64_t(s) * 64)[(i < 8 ? 0 : 8) + plane_pos(d)] = word;
    } else if (i == 16) {
        const float scale = amax * (1.f / 16383.f);
        reinterpret_cast<float *>(image_row + int64_t(S) * 64)[s] = scale;
        reinterpret_cast<float *>(image_row + int64_t(S) * 68)[s] = float(qs) * scale;
    }
}

// One wave per row: the row's maximum first, then every sub-block against it, so that all sub-blocks of a row share one
// scale (the products can then keep integer sums across sub-blocks and apply the row's scale once).
template <int XT> __device__ __forceinline__ void load_block32(const void * __restrict__ x, int64_t at, float (&v)[32]) {
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        float t[8];
        load8<XT>(x, at + 8 * c, t);
#pragma unroll
        for (int j = 0; j < 8; ++j) v[8 * c + j] = t[j];
    }
}
template <int XT> __device__ __forceinline__ void quantise_row_wave(const void * __restrict__ x, int64_t row, int cols, uint8_t * image_row, int lane) {
    const int S = cols / 32;
    float amax = 0.f;
    for (int s = lane; s < S; s += 64) {
        float v[32];
        load_block32<XT>(x, row * cols + 32 * s, v);
        amax = fmaxf(amax, block_amax(v));
    }
    amax = wave_max(amax);
    for (int s = lane; s < S; s += 64) {
        float v[32];
        load_block32<XT>(x, row * cols + 32 * s, v);
        quantise_block(v, image_row, S, s, amax);
    }
}
// row_map (may be null): image row i is made of input row row_map[i]; a negative entry leaves the image row as it is
template <int XT>
__global__ __launch_bounds__(256) void quant_act_k(const void * __restrict__ x, int n, int cols, uint8_t * __restrict__ image, const int * __restrict__ row_map = nullptr) {
    const int64_t row = int64_t(blockIdx.x) * 4 + (threadIdx.x >> 6);
    if (row >= n) return;
    const int64_t src = row_map ? row_map[row] : row;
    if (src < 0) return;
    quantise_row_wave<XT>(x, src, cols, image + row * int64_t(cols / 32) * kImageSubBytes, threadIdx.x & 63);
}

}  // namespace
}  // namespace tqmoe

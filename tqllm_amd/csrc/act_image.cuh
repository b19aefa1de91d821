// The activation image the decode products read (layout: include/tqmoe.h) and its quantiser.
#pragma once
#include "common.cuh"

namespace tqmoe {
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

}  // namespace
}  // namespace tqmoe

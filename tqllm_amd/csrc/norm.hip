// The step in front of the layer: residual add and RMS norm of the rows the router and the experts read.
//
// The reference does it in two launches over bf16 rows (Qwen35Engine::ffn_block, qwen35_forward.cpp:1114-1115):
// add_sumsq (quant_tq3.inc:303-313: m = bf16(m + r) in place, sums of squares of the rounded values per 256 elements)
// and norm_h (quant.cu:647-661: inv = rsqrt(sum / hidden + eps), y = bf16((m * inv) * w) stored as fp16). Here one wave
// owns a row: it reads both inputs once with 16-byte loads, keeps the sum in registers, reduces the squares across the
// wave, and writes the updated residual stream and the normed row. The sum of squares is accumulated per lane and then
// across lanes, which is not the reference's order; the normed values are rounded to bf16, so the two orders differ by
// at most one bf16 step, and only where a value sits on a rounding boundary.
#include "common.cuh"

namespace tqmoe {
namespace {

__device__ __forceinline__ float wave_sum(float v) {
    v += dpp_f<kDppXor1>(v);
    v += dpp_f<kDppXor2>(v);
    v += dpp_f<kDppHalfMirror>(v);
    v += dpp_f<kDppMirror>(v);
    v += __shfl_xor(v, 16, 64);
    v += __shfl_xor(v, 32, 64);
    return v;
}

__device__ __forceinline__ uint32_t pack_bf16(float a, float b) { return uint32_t(float_to_bf16_bits(a)) | uint32_t(float_to_bf16_bits(b)) << 16; }

// GPL = groups of 8 values per lane held in registers (hidden = 512 GPL); 0 = any hidden that is a multiple of 8, the
// row read twice
template <int NT, int GPL>
__global__ __launch_bounds__(256) void add_rmsnorm_k(uint16_t * __restrict__ rows, const uint16_t * __restrict__ residual, const float * __restrict__ weight,
                                                       float eps, void * __restrict__ normed, int hidden, int n) {
    const int lane = threadIdx.x & 63, row = int(blockIdx.x) * 4 + (threadIdx.x >> 6);
    if (row >= n) return;
    const int64_t at = int64_t(row) * hidden;
    const int groups = hidden / 8;
    auto sum_of = [&](int gi, float (&v)[8]) {   // v = bf16(m + r), written back when there is a residual
        load8<TQMOE_BF16>(rows, at + gi * 8, v);
        if (residual) {
            float r[8];
            load8<TQMOE_BF16>(residual, at + gi * 8, r);
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] = bf16_bits_to_float(float_to_bf16_bits(v[j] + r[j]));
            *reinterpret_cast<uint4 *>(rows + at + gi * 8) = make_uint4(pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3]), pack_bf16(v[4], v[5]), pack_bf16(v[6], v[7]));
        }
    };
    auto store = [&](int gi, const float (&v)[8], float inv) {
        const float4 w0 = *reinterpret_cast<const float4 *>(weight + gi * 8), w1 = *reinterpret_cast<const float4 *>(weight + gi * 8 + 4);
        const float w[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
        float y[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) y[j] = bf16_bits_to_float(float_to_bf16_bits(__fmul_rn(__fmul_rn(v[j], inv), w[j])));   // rounded to bf16 whatever the storage
        if constexpr (NT == TQMOE_BF16) {
            *reinterpret_cast<uint4 *>(static_cast<uint16_t *>(normed) + at + gi * 8) =
                make_uint4(pack_bf16(y[0], y[1]), pack_bf16(y[2], y[3]), pack_bf16(y[4], y[5]), pack_bf16(y[6], y[7]));
        } else {
            uint32_t h[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) h[j] = uint32_t(__half_as_ushort(__float2half_rn(y[2 * j]))) | uint32_t(__half_as_ushort(__float2half_rn(y[2 * j + 1]))) << 16;
            *reinterpret_cast<uint4 *>(static_cast<uint16_t *>(normed) + at + gi * 8) = make_uint4(h[0], h[1], h[2], h[3]);
        }
    };
    if constexpr (GPL > 0) {
        float v[GPL][8];
        float ss = 0.f;
#pragma unroll
        for (int q = 0; q < GPL; ++q) {
            sum_of(lane + 64 * q, v[q]);
#pragma unroll
            for (int j = 0; j < 8; ++j) ss += v[q][j] * v[q][j];
        }
        const float inv = rsqrtf(wave_sum(ss) / float(hidden) + eps);
#pragma unroll
        for (int q = 0; q < GPL; ++q) store(lane + 64 * q, v[q], inv);
    } else {
        float ss = 0.f;
        for (int gi = lane; gi < groups; gi += 64) {
            float v[8];
            sum_of(gi, v);
#pragma unroll
            for (int j = 0; j < 8; ++j) ss += v[j] * v[j];
        }
        const float inv = rsqrtf(wave_sum(ss) / float(hidden) + eps);
        for (int gi = lane; gi < groups; gi += 64) {
            float v[8];
            load8<TQMOE_BF16>(rows, at + gi * 8, v);   // the lane's own store above, or the untouched input
            store(gi, v, inv);
        }
    }
}

template <int NT>
void launch_add_rmsnorm(uint16_t * rows, const uint16_t * residual, const float * weight, float eps, void * normed, int hidden, int n, hipStream_t s) {
    const unsigned blocks = unsigned((n + 3) / 4);
    switch (hidden) {
        case 512: add_rmsnorm_k<NT, 1><<<blocks, 256, 0, s>>>(rows, residual, weight, eps, normed, hidden, n); break;
        case 1024: add_rmsnorm_k<NT, 2><<<blocks, 256, 0, s>>>(rows, residual, weight, eps, normed, hidden, n); break;
        case 2048: add_rmsnorm_k<NT, 4><<<blocks, 256, 0, s>>>(rows, residual, weight, eps, normed, hidden, n); break;
        case 4096: add_rmsnorm_k<NT, 8><<<blocks, 256, 0, s>>>(rows, residual, weight, eps, normed, hidden, n); break;
        default: add_rmsnorm_k<NT, 0><<<blocks, 256, 0, s>>>(rows, residual, weight, eps, normed, hidden, n); break;
    }
}

}  // namespace
}  // namespace tqmoe

using namespace tqmoe;

extern "C" int32_t tqmoe_add_rmsnorm(void * rows, const void * residual, const float * weight, float eps, void * normed, uint32_t ntype, int32_t hidden,
                                     int32_t n, void * stream, tqmoe_error * err) {
    if (!rows || !weight || !normed || hidden <= 0 || hidden % 8 || n <= 0) return fail(err, TQMOE_E_ARG, "tqmoe_add_rmsnorm: invalid shape or pointer");
    if (ntype != TQMOE_BF16 && ntype != TQMOE_F16) return fail(err, TQMOE_E_UNSUPPORTED, "tqmoe_add_rmsnorm: the normed rows are BF16 or F16");
    if (int32_t rc = need_device(err, "tqmoe_add_rmsnorm")) return rc;
    const hipStream_t s = static_cast<hipStream_t>(stream);
    if (ntype == TQMOE_BF16) launch_add_rmsnorm<TQMOE_BF16>(static_cast<uint16_t *>(rows), static_cast<const uint16_t *>(residual), weight, eps, normed, hidden, n, s);
    else launch_add_rmsnorm<TQMOE_F16>(static_cast<uint16_t *>(rows), static_cast<const uint16_t *>(residual), weight, eps, normed, hidden, n, s);
    return launched(err, "tqmoe_add_rmsnorm");
}

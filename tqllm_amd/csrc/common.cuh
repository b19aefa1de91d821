// Shared device helpers of the tqmoe library (gfx950, wave64).
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>

#include <atomic>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <set>
#include <utility>

#include "../../include/tqmoe.h"

namespace tqmoe {

// ------------------------------------------------------------------------------------------------- host side
inline int32_t fail(tqmoe_error * err, int32_t code, const char * fmt, ...) {
    if (err && err->struct_size >= sizeof(tqmoe_error)) {
        err->code = code;
        va_list ap;
        va_start(ap, fmt);
        vsnprintf(err->message, sizeof(err->message), fmt, ap);
        va_end(ap);
    }
    return code;
}
inline int32_t ok(tqmoe_error * err) {
    if (err && err->struct_size >= sizeof(tqmoe_error)) { err->code = 0; err->message[0] = 0; }
    return 0;
}
// after a launch: the launch error, if any, as TQMOE_E_DEVICE
inline int32_t launched(tqmoe_error * err, const char * what) {
    const hipError_t rc = hipGetLastError();
    if (rc != hipSuccess) return fail(err, TQMOE_E_DEVICE, "%s: %s", what, hipGetErrorString(rc));
    return ok(err);
}
// a usable device must be current; there is no CPU path behind any entry point
inline int32_t need_device(tqmoe_error * err, const char * what) {
    int dev = -1;
    const hipError_t rc = hipGetDevice(&dev);
    if (rc != hipSuccess || dev < 0) {
        (void)hipGetLastError();
        return fail(err, TQMOE_E_DEVICE, "%s: no HIP device (%s); this library has no CPU path", what,
                    rc != hipSuccess ? hipGetErrorString(rc) : "none current");
    }
    return 0;
}
// Per-device facts and one-time settings. The library keeps no state a caller could observe; these only remember what has
// already been asked of the runtime, per device, so that repeated launches do not ask again.
inline int current_device() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0) { (void)hipGetLastError(); dev = 0; }
    return dev;
}
inline int cu_count() {   // compute units of the current device
    static std::atomic<int> known[64];
    const int dev = current_device() & 63;
    int n = known[dev].load(std::memory_order_relaxed);
    if (n <= 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) { (void)hipGetLastError(); n = 256; }
        known[dev].store(n, std::memory_order_relaxed);
    }
    return n;
}
// raises a kernel's dynamic LDS limit, once per kernel and device
inline void allow_dynamic_lds(const void * kernel, int bytes) {
    static std::mutex guard;
    static std::set<std::pair<const void *, int>> done;
    const std::pair<const void *, int> key(kernel, current_device());
    std::lock_guard<std::mutex> lock(guard);
    if (done.count(key)) return;
    (void)hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    done.insert(key);
}

inline bool is_act_type(uint32_t t) { return t == TQMOE_F32 || t == TQMOE_F16 || t == TQMOE_BF16; }
inline bool is_bank_type(uint32_t t) { return t == TQMOE_Q2_K || t == TQMOE_IQ1_S || t == TQMOE_Q4_0 || t == TQMOE_Q3_K || t == TQMOE_IQ2_XXS || t == TQMOE_IQ2_XS || t == TQMOE_Q4_K || t == TQMOE_IQ3_S || t == TQMOE_IQ4_XS || t == TQMOE_NVFP4G || t == TQMOE_IQ4_NL || t == TQMOE_Q8_0 ||
           t == TQMOE_Q5_K || t == TQMOE_Q6_K || t == TQMOE_IQ3_XXS || t == TQMOE_IQ2_S;
}
inline size_t elem_bytes(uint32_t t) { return t == TQMOE_F32 ? 4 : 2; }
inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

// ----------------------------------------------------------------------------------------------- device side
constexpr int kWave = 64;

// The optional clamp of the SwiGLU inputs (MoeConfig::swiglu_clamp, src/experts/moe.hpp:34-36; moe_expert_ffn,
// src/experts/moe.cpp:128-143): limit <= 1e-6 is no clamp; else up goes to [-limit, limit] and either the gate to
// (-inf, limit] before the activation (gate_first, the GLM branch) or silu(gate) to (-inf, limit] after it.
struct Glu { float limit; int gate_first; };
__device__ __forceinline__ void glu_clamp_inputs(const Glu c, float & g, float & u) {
    if (c.limit > 1e-6f) {
        u = fminf(fmaxf(u, -c.limit), c.limit);
        if (c.gate_first) g = fminf(g, c.limit);
    }
}
__device__ __forceinline__ float glu_clamp_silu(const Glu c, float s) { return c.limit > 1e-6f && !c.gate_first ? fminf(s, c.limit) : s; }

__device__ __forceinline__ float bf16_bits_to_float(uint16_t h) { return __uint_as_float(uint32_t(h) << 16); }
__device__ __forceinline__ uint16_t float_to_bf16_bits(float f) {  // round to nearest even
    const uint32_t x = __float_as_uint(f);
    if ((x & 0x7FFFFFFFu) > 0x7F800000u) return uint16_t((x >> 16) | 0x40u);
    return uint16_t((x + 0x7FFFu + ((x >> 16) & 1u)) >> 16);
}
__device__ __forceinline__ float half_bits_to_float(uint16_t h) { return __half2float(__ushort_as_half(h)); }

template <int TYPE> struct Elem;
template <> struct Elem<TQMOE_F32> {
    using type = float;
    static __device__ __forceinline__ float get(const void * p, int64_t i) { return static_cast<const float *>(p)[i]; }
};
template <> struct Elem<TQMOE_F16> {
    using type = uint16_t;
    static __device__ __forceinline__ float get(const void * p, int64_t i) { return half_bits_to_float(static_cast<const uint16_t *>(p)[i]); }
};
template <> struct Elem<TQMOE_BF16> {
    using type = uint16_t;
    static __device__ __forceinline__ float get(const void * p, int64_t i) { return bf16_bits_to_float(static_cast<const uint16_t *>(p)[i]); }
};

// 8 consecutive elements starting at a multiple of 8, as floats
template <int TYPE> __device__ __forceinline__ void load8(const void * p, int64_t i, float (&v)[8]) {
    if constexpr (TYPE == TQMOE_F32) {
        const float4 a = *reinterpret_cast<const float4 *>(static_cast<const float *>(p) + i);
        const float4 b = *reinterpret_cast<const float4 *>(static_cast<const float *>(p) + i + 4);
        v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
    } else {
        const uint4 q = *reinterpret_cast<const uint4 *>(static_cast<const uint16_t *>(p) + i);
        const uint32_t w[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if constexpr (TYPE == TQMOE_BF16) {
                v[2 * j] = __uint_as_float(w[j] << 16);
                v[2 * j + 1] = __uint_as_float(w[j] & 0xFFFF0000u);
            } else {
                v[2 * j] = half_bits_to_float(uint16_t(w[j] & 0xFFFFu));
                v[2 * j + 1] = half_bits_to_float(uint16_t(w[j] >> 16));
            }
        }
    }
}

template <int TYPE> __device__ __forceinline__ void store_out(void * p, int64_t i, float v) {
    if constexpr (TYPE == TQMOE_F32) static_cast<float *>(p)[i] = v;
    else if constexpr (TYPE == TQMOE_BF16) static_cast<uint16_t *>(p)[i] = float_to_bf16_bits(v);
    else static_cast<uint16_t *>(p)[i] = __half_as_ushort(__float2half_rn(v));
}

// DPP lane exchange inside a row of 16 lanes
template <int CTRL> __device__ __forceinline__ float dpp_f(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}
template <int CTRL> __device__ __forceinline__ int dpp_i(int v) { return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xF, 0xF, true); }
constexpr int kDppXor1 = 0xB1;          // quad_perm [1,0,3,2]
constexpr int kDppXor2 = 0x4E;          // quad_perm [2,3,0,1]
constexpr int kDppHalfMirror = 0x141;   // lane i <-> 7 - i inside 8
constexpr int kDppMirror = 0x140;       // lane i <-> 15 - i inside 16

// sum over each row of 16 lanes, in every lane of the row
__device__ __forceinline__ float row_sum16(float v) {
    v += dpp_f<kDppXor1>(v);
    v += dpp_f<kDppXor2>(v);
    v += dpp_f<kDppHalfMirror>(v);
    v += dpp_f<kDppMirror>(v);
    return v;
}

// all-reduce sum over groups of WIDTH consecutive lanes (WIDTH a power of two, 1..64); every lane gets the total
template <int WIDTH> __device__ __forceinline__ float group_sum(float v) {
    if constexpr (WIDTH >= 2) v += dpp_f<kDppXor1>(v);
    if constexpr (WIDTH >= 4) v += dpp_f<kDppXor2>(v);
    if constexpr (WIDTH >= 8) v += dpp_f<kDppHalfMirror>(v);
    if constexpr (WIDTH >= 16) v += dpp_f<kDppMirror>(v);
    if constexpr (WIDTH >= 32) v += __shfl_xor(v, 16, 64);
    if constexpr (WIDTH >= 64) v += __shfl_xor(v, 32, 64);
    return v;
}
__device__ __forceinline__ float group_sum_rt(float v, int width) {  // run-time width
    switch (width) {
        case 1: return v;
        case 2: return group_sum<2>(v);
        case 4: return group_sum<4>(v);
        case 8: return group_sum<8>(v);
        case 16: return group_sum<16>(v);
        case 32: return group_sum<32>(v);
        default: return group_sum<64>(v);
    }
}
__device__ __forceinline__ float wave_max(float v) {
    v = fmaxf(v, dpp_f<kDppXor1>(v));
    v = fmaxf(v, dpp_f<kDppXor2>(v));
    v = fmaxf(v, dpp_f<kDppHalfMirror>(v));
    v = fmaxf(v, dpp_f<kDppMirror>(v));
    v = fmaxf(v, __shfl_xor(v, 16, 64));
    v = fmaxf(v, __shfl_xor(v, 32, 64));
    return v;
}

}  // namespace tqmoe

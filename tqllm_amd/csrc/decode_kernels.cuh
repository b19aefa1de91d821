// Decode-sized expert products: the kernels and their per-format launch tables (one translation unit per bank format
// instantiates DecodeLaunch<FMT>; decode.hip holds the entry points).
//
// HBM-streaming matrix-vector kernels over the bank layout.
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
#pragma once
#include "act_image.cuh"
#include "decode_api.cuh"
#include "formats.cuh"

namespace tqmoe {
namespace {

// ------------------------------------------------------------------------------------------ sub-block products
// A weight sub-block is fetched (Raw: what one lane loads), decoded once into eight dwords of int8 values in the order
// of the activation planes (Dec), and multiplied with any number of activation blocks.
struct Dec {
    uint32_t w[8];   // int8 x 4 each; w[q] = values 4q .. 4q + 3 of the sub-block
    float s0, s1;    // scale of dwords 0..3 and of dwords 4..7 (equal unless the format scales 16-weight groups)
    float mn;        // coefficient of the block's activation sum (a K-quant minimum), else 0; with half minimums (Q2_K): of
    float mn1;       // the first 16 weights' sum, and mn1 of the other 16's
};

// w: natural dwords d0 .. d0 + 3 of a sub-block's values; x: a plane indexed by plane position
template <int D0> __device__ __forceinline__ int dot4x(const uint32_t * w, const int * x) {
    int acc = 0;
#pragma unroll
    for (int q = 0; q < 4; ++q) acc = __builtin_amdgcn_sdot4(int(w[q]), x[plane_pos(D0 + q)], acc, false);
    return acc;
}
// a format whose traits declare kHalfMins has a minimum per 16 weights
template <class F, class = void> struct HalfMins { static constexpr bool value = false; };
template <class F> struct HalfMins<F, decltype(void(F::kHalfMins))> { static constexpr bool value = true; };

template <bool SPLIT, bool HALF_MINS = false> __device__ __forceinline__ float dot_block(const Dec & d, const ActBlock & x) {
    if constexpr (HALF_MINS) {
        const int t0 = (dot4x<0>(d.w, x.hi) << 7) + dot4x<0>(d.w, x.lo);
        const int t1 = (dot4x<4>(d.w + 4, x.hi) << 7) + dot4x<4>(d.w + 4, x.lo);
        const uint32_t ones[4] = {0x01010101u, 0x01010101u, 0x01010101u, 0x01010101u};
        const float u0 = float((dot4x<0>(ones, x.hi) << 7) + dot4x<0>(ones, x.lo)) * x.scale;   // the first half's activation sum
        return (float(t0) * d.s0 + float(t1) * d.s1) * x.scale - d.mn * u0 - d.mn1 * (x.sum - u0);
    } else if constexpr (SPLIT) {
        const int t0 = (dot4x<0>(d.w, x.hi) << 7) + dot4x<0>(d.w, x.lo);
        const int t1 = (dot4x<4>(d.w + 4, x.hi) << 7) + dot4x<4>(d.w + 4, x.lo);
        return (float(t0) * d.s0 + float(t1) * d.s1) * x.scale;
    } else {
        int hi = 0, lo = 0;
#pragma unroll
        for (int q = 0; q < 8; ++q) {
            hi = __builtin_amdgcn_sdot4(int(d.w[q]), x.hi[plane_pos(q)], hi, false);
            lo = __builtin_amdgcn_sdot4(int(d.w[q]), x.lo[plane_pos(q)], lo, false);
        }
        return float((hi << 7) + lo) * (d.s0 * x.scale) - d.mn * x.sum;
    }
}

// Uniform base pointers of one bank for the rows [row0, ...) of expert e: lanes add 32-bit offsets to them.
struct Tile { const uint8_t * codes; const uint8_t * aux; const uint8_t * aux2; };
template <uint32_t FMT> __device__ __forceinline__ Tile tile_of(const BankView & b, int e, int row0) {
    const int64_t row = int64_t(e) * b.rows + row0;
    Tile t;
    t.codes = b.codes + row * code_row_bytes(FMT, b.cols);
    t.aux = b.aux + row * aux_row_bytes(FMT, b.cols);
    t.aux2 = FMT == TQMOE_NVFP4G ? b.aux + nvfp4_global_offset(b.rows_total, b.cols) + row * 4 : nullptr;
    return t;
}

template <uint32_t FMT> struct Sub;

template <> struct Sub<TQMOE_Q4_K> {
    static constexpr bool kSplit = false;
    struct Raw { uint4 c; uint4 rec; };
    static __device__ __forceinline__ Raw load(const Tile & t, uint32_t r, uint32_t S, uint32_t s) {
        Raw v;
        v.c = *reinterpret_cast<const uint4 *>(t.codes + (r * S + s) * 16u);
        v.rec = *reinterpret_cast<const uint4 *>(t.aux + (r * (S >> 3) + (s >> 3)) * 16u);
        return v;
    }
    static __device__ __forceinline__ void decode(const Raw & r, int s, const uint32_t *, Dec & d) {
        const uint32_t w[4] = {r.c.x, r.c.y, r.c.z, r.c.w};
#pragma unroll
        for (int q = 0; q < 4; ++q) nibbles(w[q], d.w[q], d.w[4 + q]);
        const uint32_t sc12[3] = {r.rec.y, r.rec.z, r.rec.w};
        int sc, mn;
        q4k_scale_min(sc12, s & 7, sc, mn);
        d.s0 = d.s1 = half_bits_to_float(uint16_t(r.rec.x & 0xFFFFu)) * float(sc);
        d.mn = half_bits_to_float(uint16_t(r.rec.x >> 16)) * float(mn);
    }
};

template <> struct Sub<TQMOE_IQ3_XXS> {
    static constexpr bool kSplit = false;
    struct Raw { uint32_t c[3]; uint32_t d; };
    static __device__ __forceinline__ Raw load(const Tile & t, uint32_t r, uint32_t S, uint32_t s) {
        Raw v;
        const uint32_t * cp = reinterpret_cast<const uint32_t *>(t.codes + (r * S + s) * 12u);
        v.c[0] = cp[0]; v.c[1] = cp[1]; v.c[2] = cp[2];
        v.d = *reinterpret_cast<const uint16_t *>(t.aux + (r * (S >> 3) + (s >> 3)) * 16u);
        return v;
    }
    // grid: the 256-entry lattice in LDS
    static __device__ __forceinline__ void decode(const Raw & r, int, const uint32_t * grid, Dec & d) {
#pragma unroll
        for (int w = 0; w < 8; ++w) {
            const uint32_t g = grid[(r.c[w >> 2] >> (8 * (w & 3))) & 0xFFu];
            const uint32_t bits = spread4(iq3xxs_signs(r.c[2], w >> 1) >> (4 * (w & 1)));
            const uint32_t m = (bits << 8) - bits;   // byte masks 0xFF; negate the selected bytes: (g ^ m) + bits, no carry leaves a byte
            d.w[w] = (g ^ m) + bits;
        }
        d.s0 = d.s1 = half_bits_to_float(uint16_t(r.d)) * (0.5f + float(r.c[2] >> 28)) * 0.5f;
        d.mn = 0.f;
    }
};

template <> struct Sub<TQMOE_IQ2_S> {
    static constexpr bool kSplit = true;   // one scale nibble per 16 weights: the sub-block's halves
    struct Raw { uint32_t c[3]; uint32_t d; };
    static __device__ __forceinline__ Raw load(const Tile & t, uint32_t r, uint32_t S, uint32_t s) {
        Raw v;
        const uint32_t * cp = reinterpret_cast<const uint32_t *>(t.codes + (r * S + s) * 12u);
        v.c[0] = cp[0]; v.c[1] = cp[1]; v.c[2] = cp[2];
        v.d = *reinterpret_cast<const uint16_t *>(t.aux + (r * (S >> 3) + (s >> 3)) * 16u);
        return v;
    }
    // grid: the 1024-point lattice in LDS, two dwords per point
    static __device__ __forceinline__ void decode(const Raw & r, int, const uint32_t * grid, Dec & d) {
        const uint32_t qh = r.c[2] & 0xFFu, sc = (r.c[2] >> 8) & 0xFFu;
#pragma unroll
        for (int w = 0; w < 8; ++w) {   // group l = w / 2 of eight weights, half h = w % 2
            const uint32_t g = grid[2 * iq2s_index(r.c[0], qh, w >> 1) + (w & 1)];
            const uint32_t bits = spread4(r.c[1] >> (8 * (w >> 1) + 4 * (w & 1)));
            const uint32_t m = (bits << 8) - bits;
            d.w[w] = (g ^ m) + bits;
        }
        const float dd = half_bits_to_float(uint16_t(r.d));
        d.s0 = dd * (0.5f + float(sc & 15u)) * 0.25f;
        d.s1 = dd * (0.5f + float(sc >> 4)) * 0.25f;
        d.mn = 0.f;
    }
};

template <> struct Sub<TQMOE_IQ2_XXS> {
    static constexpr bool kSplit = false;
    struct Raw { uint2 c; uint32_t d; };
    static __device__ __forceinline__ Raw load(const Tile & t, uint32_t r, uint32_t S, uint32_t s) {
        Raw v;
        v.c = *reinterpret_cast<const uint2 *>(t.codes + (r * S + s) * 8u);
        v.d = *reinterpret_cast<const uint16_t *>(t.aux + (r * (S >> 3) + (s >> 3)) * 16u);
        return v;
    }
    // grid: the 256-point lattice in LDS, two dwords per point
    static __device__ __forceinline__ void decode(const Raw & r, int, const uint32_t * grid, Dec & d) {
#pragma unroll
        for (int l = 0; l < 4; ++l) {
            const uint2 g = *reinterpret_cast<const uint2 *>(grid + 2u * ((r.c.x >> (8 * l)) & 0xFFu));
            const uint32_t sn = iq3xxs_signs(r.c.y, l);
            d.w[2 * l] = apply_signs4(g.x, sn);
            d.w[2 * l + 1] = apply_signs4(g.y, sn >> 4);
        }
        d.s0 = d.s1 = half_bits_to_float(uint16_t(r.d)) * (0.5f + float(r.c.y >> 28)) * 0.25f;
        d.mn = 0.f;
    }
};

template <> struct Sub<TQMOE_IQ2_XS> {
    static constexpr bool kSplit = true;   // one scale nibble per 16 weights: the sub-block's halves
    struct Raw { uint32_t c[3]; uint32_t d; };
    static __device__ __forceinline__ Raw load(const Tile & t, uint32_t r, uint32_t S, uint32_t s) {
        Raw v;
        const uint32_t * cp = reinterpret_cast<const uint32_t *>(t.codes + (r * S + s) * 12u);
        v.c[0] = cp[0]; v.c[1] = cp[1]; v.c[2] = cp[2];
        v.d = *reinterpret_cast<const uint16_t *>(t.aux + (r * (S >> 3) + (s >> 3)) * 16u);
        return v;
    }
    // grid: the 512-point lattice in LDS, two dwords per point
    static __device__ __forceinline__ void decode(const Raw & r, int, const uint32_t * grid, Dec & d) {
#pragma unroll
        for (int l = 0; l < 4; ++l) {
            const uint32_t q = (r.c[l >> 1] >> (16 * (l & 1))) & 0xFFFFu;
            const uint2 g = *reinterpret_cast<const uint2 *>(grid + 2u * (q & 511u));
            const uint32_t sn = signs8(q >> 9);
            d.w[2 * l] = apply_signs4(g.x, sn);
            d.w[2 * l + 1] = apply_signs4(g.y, sn >> 4);
        }
        const float dd = half_bits_to_float(uint16_t(r.d));
        d.s0 = dd * (0.5f + float(r.c[2] & 15u)) * 0.25f;
        d.s1 = dd * (0.5f + float((r.c[2] >> 4) & 15u)) * 0.25f;
        d.mn = 0.f;
    }
};

template <> struct Sub<TQMOE_Q3_K> {
    static constexpr bool kSplit = true;   // one scale per 16 weights: the sub-block's halves
    struct Raw { uint32_t c[3]; uint32_t sc; uint32_t d; };
    static __device__ __forceinline__ Raw load(const Tile & t, uint32_t r, uint32_t S, uint32_t s) {
        Raw v;
        const uint32_t * cp = reinterpret_cast<const uint32_t *>(t.codes + (r * S + s) * 12u);
        v.c[0] = cp[0]; v.c[1] = cp[1]; v.c[2] = cp[2];
        const uint8_t * a = t.aux + (r * (S >> 3) + (s >> 3)) * 32u;
        v.sc = *reinterpret_cast<const uint16_t *>(a + 2u * (s & 7u));
        v.d = *reinterpret_cast<const uint16_t *>(a + 16u);
        return v;
    }
    static __device__ __forceinline__ void decode(const Raw & r, int, const uint32_t *, Dec & d) {
#pragma unroll
        for (int q = 0; q < 8; ++q)   // weights 4 q ..: two low bits from byte q of the low plane, the third from four mask bits
            d.w[q] = minus_k<4>(spread2x4(r.c[q >> 2] >> (8 * (q & 3))) | spread4(r.c[2] >> (4 * q)) << 2);
        const float dd = half_bits_to_float(uint16_t(r.d));
        d.s0 = dd * float(int8_t(r.sc & 0xFFu));
        d.s1 = dd * float(int8_t(r.sc >> 8));
        d.mn = 0.f;
    }
};

template <> struct Sub<TQMOE_Q2_K> {
    static constexpr bool kSplit = true;      // one scale and one minimum per 16 weights: the sub-block's halves
    static constexpr bool kHalfMins = true;
    struct Raw { uint2 c; uint32_t sc; uint32_t dm; };
    static __device__ __forceinline__ Raw load(const Tile & t, uint32_t r, uint32_t S, uint32_t s) {
        Raw v;
        v.c = *reinterpret_cast<const uint2 *>(t.codes + (r * S + s) * 8u);
        const uint8_t * a = t.aux + (r * (S >> 3) + (s >> 3)) * 32u;
        v.sc = *reinterpret_cast<const uint16_t *>(a + 2u * (s & 7u));
        v.dm = *reinterpret_cast<const uint32_t *>(a + 16u);
        return v;
    }
    static __device__ __forceinline__ void decode(const Raw & r, int, const uint32_t *, Dec & d) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            d.w[q] = spread2x4(r.c.x >> (8 * q));
            d.w[4 + q] = spread2x4(r.c.y >> (8 * q));
        }
        const float dd = half_bits_to_float(uint16_t(r.dm & 0xFFFFu)), dmin = half_bits_to_float(uint16_t(r.dm >> 16));
        d.s0 = dd * float(r.sc & 15u);
        d.s1 = dd * float((r.sc >> 8) & 15u);
        d.mn = dmin * float((r.sc >> 4) & 15u);
        d.mn1 = dmin * float((r.sc >> 12) & 15u);
    }
};

template <> struct Sub<TQMOE_IQ1_S> {
    static constexpr bool kSplit = false;
    struct Raw { uint2 c; uint32_t d; };
    static __device__ __forceinline__ Raw load(const Tile & t, uint32_t r, uint32_t S, uint32_t s) {
        Raw v;
        v.c = *reinterpret_cast<const uint2 *>(t.codes + (r * S + s) * 8u);
        v.d = *reinterpret_cast<const uint16_t *>(t.aux + (r * (S >> 3) + (s >> 3)) * 16u);
        return v;
    }
    // grid: the 2048-point lattice in LDS, two dwords per point of int8 values; value + delta is split into the integer
    // product and delta times the block's activation sum
    static __device__ __forceinline__ void decode(const Raw & r, int, const uint32_t * grid, Dec & d) {
#pragma unroll
        for (int l = 0; l < 4; ++l) {
            const uint2 g = *reinterpret_cast<const uint2 *>(grid + 2u * (((r.c.x >> (8 * l)) & 0xFFu) | (((r.c.y >> (3 * l)) & 7u) << 8)));
            d.w[2 * l] = g.x;
            d.w[2 * l + 1] = g.y;
        }
        d.s0 = d.s1 = half_bits_to_float(uint16_t(r.d)) * float(2 * int((r.c.y >> 12) & 7u) + 1);
        d.mn = (r.c.y & 0x8000u) ? 0.125f * d.s0 : -0.125f * d.s0;
    }
};

template <> struct Sub<TQMOE_Q4_0> {
    static constexpr bool kSplit = false;
    struct Raw { uint4 c; uint32_t d; };
    static __device__ __forceinline__ Raw load(const Tile & t, uint32_t r, uint32_t S, uint32_t s) {
        Raw v;
        v.c = *reinterpret_cast<const uint4 *>(t.codes + (r * S + s) * 16u);
        v.d = *reinterpret_cast<const uint16_t *>(t.aux + (r * S + s) * 2u);
        return v;
    }
    static __device__ __forceinline__ void decode(const Raw & r, int, const uint32_t *, Dec & d) {
        const uint32_t w[4] = {r.c.x, r.c.y, r.c.z, r.c.w};
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            uint32_t lo, hi;
            nibbles(w[q], lo, hi);
            d.w[q] = minus_k<8>(lo);
            d.w[4 + q] = minus_k<8>(hi);
        }
        d.s0 = d.s1 = half_bits_to_float(uint16_t(r.d));
        d.mn = 0.f;
    }
};

template <> struct Sub<TQMOE_Q5_K> {
    static constexpr bool kSplit = false;
    struct Raw { uint4 c; uint4 rec; uint32_t hb; };
    static __device__ __forceinline__ Raw load(const Tile & t, uint32_t r, uint32_t S, uint32_t s) {
        Raw v;
        v.c = *reinterpret_cast<const uint4 *>(t.codes + (r * S + s) * 16u);
        const uint8_t * a = t.aux + (r * (S >> 3) + (s >> 3)) * 48u;
        v.rec = *reinterpret_cast<const uint4 *>(a);
        v.hb = *reinterpret_cast<const uint32_t *>(a + 16u + 4u * (s & 7u));
        return v;
    }
    static __device__ __forceinline__ void decode(const Raw & r, int s, const uint32_t *, Dec & d) {
        const uint32_t w[4] = {r.c.x, r.c.y, r.c.z, r.c.w};
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            nibbles(w[q], d.w[q], d.w[4 + q]);
            d.w[q] |= spread4(r.hb >> (4 * q)) << 4;            // the fifth bit of weights 4 q ..
            d.w[4 + q] |= spread4(r.hb >> (16 + 4 * q)) << 4;   // and of weights 16 + 4 q ..
        }
        const uint32_t sc12[3] = {r.rec.y, r.rec.z, r.rec.w};
        int sc, mn;
        q4k_scale_min(sc12, s & 7, sc, mn);
        d.s0 = d.s1 = half_bits_to_float(uint16_t(r.rec.x & 0xFFFFu)) * float(sc);
        d.mn = half_bits_to_float(uint16_t(r.rec.x >> 16)) * float(mn);
    }
};

template <> struct Sub<TQMOE_Q6_K> {
    static constexpr bool kSplit = true;   // one scale per 16 weights: the sub-block's halves
    struct Raw { uint2 c[3]; uint32_t sc; uint32_t d; };
    static __device__ __forceinline__ Raw load(const Tile & t, uint32_t r, uint32_t S, uint32_t s) {
        Raw v;
        const uint2 * cp = reinterpret_cast<const uint2 *>(t.codes + (r * S + s) * 24u);
        v.c[0] = cp[0]; v.c[1] = cp[1]; v.c[2] = cp[2];
        const uint8_t * a = t.aux + (r * (S >> 3) + (s >> 3)) * 32u;
        v.sc = *reinterpret_cast<const uint16_t *>(a + 2u * (s & 7u));
        v.d = *reinterpret_cast<const uint16_t *>(a + 16u);
        return v;
    }
    static __device__ __forceinline__ void decode(const Raw & r, int, const uint32_t *, Dec & d) {
        const uint32_t w[4] = {r.c[0].x, r.c[0].y, r.c[1].x, r.c[1].y};
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            uint32_t lo, hi;
            nibbles(w[q], lo, hi);
            d.w[q] = minus32(lo | spread2x4(r.c[2].x >> (8 * q)) << 4);
            d.w[4 + q] = minus32(hi | spread2x4(r.c[2].y >> (8 * q)) << 4);
        }
        const float dd = half_bits_to_float(uint16_t(r.d));
        d.s0 = dd * float(int8_t(r.sc & 0xFFu));
        d.s1 = dd * float(int8_t(r.sc >> 8));
        d.mn = 0.f;
    }
};

template <> struct Sub<TQMOE_IQ4_NL> {
    static constexpr bool kSplit = false;
    struct Raw { uint4 c; uint32_t d; };
    static __device__ __forceinline__ Raw load(const Tile & t, uint32_t r, uint32_t S, uint32_t s) {
        Raw v;
        v.c = *reinterpret_cast<const uint4 *>(t.codes + (r * S + s) * 16u);
        v.d = *reinterpret_cast<const uint16_t *>(t.aux + (r * S + s) * 2u);
        return v;
    }
    static __device__ __forceinline__ void decode(const Raw & r, int, const uint32_t *, Dec & d) {
        const uint32_t w[4] = {r.c.x, r.c.y, r.c.z, r.c.w};
#pragma unroll
        for (int q = 0; q < 4; ++q) lookup16<kIq4T0, kIq4T1, kIq4T2, kIq4T3>(w[q], d.w[q], d.w[4 + q]);
        d.s0 = d.s1 = half_bits_to_float(uint16_t(r.d));
        d.mn = 0.f;
    }
};

template <> struct Sub<TQMOE_Q8_0> {
    static constexpr bool kSplit = false;
    struct Raw { uint4 c0, c1; uint32_t d; };
    static __device__ __forceinline__ Raw load(const Tile & t, uint32_t r, uint32_t S, uint32_t s) {
        Raw v;
        const uint4 * cp = reinterpret_cast<const uint4 *>(t.codes + (r * S + s) * 32u);
        v.c0 = cp[0]; v.c1 = cp[1];
        v.d = *reinterpret_cast<const uint16_t *>(t.aux + (r * S + s) * 2u);
        return v;
    }
    static __device__ __forceinline__ void decode(const Raw & r, int, const uint32_t *, Dec & d) {   // the codes are the values
        d.w[0] = r.c0.x; d.w[1] = r.c0.y; d.w[2] = r.c0.z; d.w[3] = r.c0.w;
        d.w[4] = r.c1.x; d.w[5] = r.c1.y; d.w[6] = r.c1.z; d.w[7] = r.c1.w;
        d.s0 = d.s1 = half_bits_to_float(uint16_t(r.d));
        d.mn = 0.f;
    }
};

template <> struct Sub<TQMOE_NVFP4G> {
    static constexpr bool kSplit = true;
    struct Raw { uint4 c; uint32_t sc; float g; };
    static __device__ __forceinline__ Raw load(const Tile & t, uint32_t r, uint32_t S, uint32_t s) {
        Raw v;
        v.c = *reinterpret_cast<const uint4 *>(t.codes + (r * S + s) * 16u);
        v.sc = *reinterpret_cast<const uint16_t *>(t.aux + (r * S + s) * 2u);
        v.g = *reinterpret_cast<const float *>(t.aux2 + r * 4u);
        return v;
    }
    static __device__ __forceinline__ void decode(const Raw & r, int, const uint32_t *, Dec & d) {
        const uint32_t w[4] = {r.c.x, r.c.y, r.c.z, r.c.w};
#pragma unroll
        for (int q = 0; q < 4; ++q) lookup16<kFp4T0, kFp4T1, kFp4T2, kFp4T3>(w[q], d.w[q], d.w[4 + q]);
        // low nibbles = the first 16-weight group, high nibbles = the second; table values are twice the E2M1 value
        d.s0 = e4m3_to_float_fast(r.sc & 0xFFu) * (0.5f * r.g);
        d.s1 = e4m3_to_float_fast(r.sc >> 8) * (0.5f * r.g);
        d.mn = 0.f;
    }
};

template <> struct Sub<TQMOE_IQ3_S> {
    static constexpr bool kSplit = false;
    struct Raw { uint32_t c[3]; uint4 rec; };
    static __device__ __forceinline__ Raw load(const Tile & t, uint32_t r, uint32_t S, uint32_t s) {
        Raw v;
        const uint32_t * cp = reinterpret_cast<const uint32_t *>(t.codes + (r * S + s) * 12u);
        v.c[0] = cp[0]; v.c[1] = cp[1]; v.c[2] = cp[2];
        v.rec = *reinterpret_cast<const uint4 *>(t.aux + (r * (S >> 3) + (s >> 3)) * 16u);
        return v;
    }
    // grid: the 512-entry lattice in LDS
    static __device__ __forceinline__ void decode(const Raw & r, int s, const uint32_t * grid, Dec & d) {
        const int ib = s & 7;
        const uint4 rec = r.rec;
        const uint32_t qh = ib < 2 ? (rec.x >> (16 + 8 * ib)) & 0xFFu : ib < 6 ? (rec.y >> (8 * (ib - 2))) & 0xFFu : (rec.z >> (8 * (ib - 6))) & 0xFFu;
        const uint32_t scb = (ib >> 1) < 2 ? (rec.z >> (16 + 8 * (ib >> 1))) & 0xFFu : (rec.w >> (8 * ((ib >> 1) - 2))) & 0xFFu;
#pragma unroll
        for (int w = 0; w < 8; ++w) {
            const uint32_t g = grid[((r.c[w >> 2] >> (8 * (w & 3))) & 0xFFu) | (((qh >> w) & 1u) << 8)];
            // four sign bits -> byte masks 0xFF; negate the selected bytes: (g ^ m) + (m & 0x01010101), no carry leaves a byte
            const uint32_t bits = (((r.c[2] >> (4 * w)) & 15u) * 0x00204081u) & 0x01010101u;
            const uint32_t m = (bits << 8) - bits;
            d.w[w] = (g ^ m) + bits;
        }
        d.s0 = d.s1 = half_bits_to_float(uint16_t(rec.x & 0xFFFFu)) * float(1 + 2 * int((scb >> (4 * (ib & 1))) & 15u));
        d.mn = 0.f;
    }
};

template <uint32_t FMT> __device__ __forceinline__ const uint32_t * stage_grid(uint32_t * lds) {
    const uint32_t * src = nullptr;
    if constexpr (FMT == TQMOE_IQ3_S) src = d_iq3s_grid.v;
    else if constexpr (FMT == TQMOE_IQ3_XXS) src = d_iq3xxs_grid.v;
    else if constexpr (FMT == TQMOE_IQ2_S) src = d_iq2s_grid.v;
    else if constexpr (FMT == TQMOE_IQ2_XS) src = d_iq2xs_grid.v;
    else if constexpr (FMT == TQMOE_IQ2_XXS) src = d_iq2xxs_grid.v;
    else if constexpr (FMT == TQMOE_IQ1_S) src = d_iq1s_grid.v;
    if constexpr (lattice_dwords(FMT) > 1) {
        for (int i = threadIdx.x; i < lattice_dwords(FMT); i += blockDim.x) lds[i] = src[i];
        __syncthreads();
        return lds;
    } else {
        return nullptr;
    }
}

// sum over the LPR consecutive lanes of a row; valid in the last lane of each group
template <int LPR> __device__ __forceinline__ float row_total(float v) {
    v += dpp_f<kDppXor1>(v);
    v += dpp_f<kDppXor2>(v);
    v += dpp_f<kDppHalfMirror>(v);
    if constexpr (LPR >= 16) v += dpp_f<kDppMirror>(v);
    if constexpr (LPR >= 32) v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x142, 0xA, 0xF, false));  // row_bcast:15
    if constexpr (LPR >= 64) v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x143, 0xC, 0xF, false));  // row_bcast:31
    return v;
}

// Pairing of the assignments that share an expert, so that their blocks read the weights once for two input rows.
// mode 0: every assignment alone. mode 1: among the assignments of ids[0..A) with this block's expert, in index order,
// the 1st, 3rd, ... each take the next one along (returns 2 and sets partner) or go alone when they are the last
// (returns 1); the 2nd, 4th, ... leave (returns 0). meta: two ints of LDS.
__device__ __forceinline__ int pair_up(const int * __restrict__ ids, int A, int a, int e, int mode, int * meta, int & partner) {
    partner = a;
    if (mode == 0) return 1;
    if (threadIdx.x == 0) { meta[0] = 0; meta[1] = 0x7FFFFFFF; }
    __syncthreads();
    for (int i = threadIdx.x; i < A; i += blockDim.x)
        if (ids[i] == e) {
            if (i < a) atomicAdd(&meta[0], 1);
            if (i > a) atomicMin(&meta[1], i);
        }
    __syncthreads();
    if (meta[0] & 1) return 0;
    if (meta[1] == 0x7FFFFFFF) return 1;
    partner = meta[1];
    return 2;
}

// Core of every decode product: one block of NW waves, rows [0, NJ * NW * (64 / LPR)) of the tiles of NB banks (the
// same rows of each), NT activation rows at a time. Lane (rl, sl) of wave w handles row (j * NW + w) * RW + rl and
// sub-blocks sl + LPR * m of it. Rows past `rows_left` are computed on the last valid row (and dropped by emit's
// caller). emit(nb, nt, row, value) runs in the last lane of each row group.
template <uint32_t FMT, int LPR, int M, int NB, int NT, int NJ, int NW, class Emit>
__device__ __forceinline__ void block_rows(const Tile (&tile)[NB], int S, int rows_left, const ActBlock (&x)[NT][M], const uint32_t * grid, Emit emit) {
    using F = Sub<FMT>;
    // row steps whose weight loads are in flight together: all four where a lane holds one sub-block per row (the block is
    // then one trip to memory and one run of products), else two
    constexpr int RW = 64 / LPR, U = (M == 1 && NJ % 4 == 0) ? 4 : (M >= 3) ? 1 : NJ >= 2 ? 2 : 1;
    static_assert(NJ % U == 0, "row steps come in pairs");
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int rl = lane / LPR, sl = lane % LPR;
    const uint32_t last = uint32_t(rows_left - 1);
#pragma unroll
    for (int j0 = 0; j0 < NJ; j0 += U) {
        typename F::Raw raw[U][NB][M];
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int nb = 0; nb < NB; ++nb)
#pragma unroll
                for (int m = 0; m < M; ++m)
                    raw[u][nb][m] = F::load(tile[nb], min(uint32_t(((j0 + u) * NW + wave) * RW + rl), last), uint32_t(S), min(uint32_t(sl + LPR * m), uint32_t(S - 1)));
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
                float acc[NT];
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) acc[nt] = 0.f;
#pragma unroll
                for (int m = 0; m < M; ++m) {
                    Dec d;
                    F::decode(raw[u][nb][m], min(sl + LPR * m, S - 1), grid, d);
#pragma unroll
                    for (int nt = 0; nt < NT; ++nt) acc[nt] += dot_block<F::kSplit, HalfMins<F>::value>(d, x[nt][m]);   // blocks past the row's end are zero
                }
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    const float tot = row_total<LPR>(acc[nt]);
                    if (sl == LPR - 1) emit(nb, nt, ((j0 + u) * NW + wave) * RW + rl, tot);
                }
            }
    }
}

// the lane's activation blocks of NT image rows; sub-blocks at or past s_end are zero
template <int M, int NT>
__device__ __forceinline__ void load_x(const uint8_t * __restrict__ image, const int (&xrow)[NT], int S, int s_end, int lpr, int sl, ActBlock (&x)[NT][M]) {
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int m = 0; m < M; ++m) {
            const int s = sl + lpr * m;
            if (s < s_end) load_act_block(image + int64_t(xrow[nt]) * S * kImageSubBytes, S, s, x[nt][m]); else zero_act_block(x[nt][m]);
        }
}

// ------------------------------------------------------------------------------------------- grouped mat-vec
// grid (row tiles, assignments), NW waves. y[a][r] for the tile's rows; NB banks (gate and up) share ids and the input.
// (IQ3_S with three sub-blocks a lane and one bank sits three registers above what lets a SIMD hold three waves: it is held to that)
template <uint32_t FMT, int LPR, int M, int NB, int NJ, int NW>
__global__ __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu((FMT == TQMOE_IQ3_S && M == 3 && NB == 1) ? 3 : 1))) void matvec_k(BankView b0, BankView b1, const uint8_t * __restrict__ image, void * y0, void * y1, uint32_t ytype,
                                                    const int * __restrict__ ids, int A, int xdiv, int mode, int slots, int topk, int shared_cols) {
    __shared__ __attribute__((aligned(8))) uint32_t grid_lds[lattice_dwords(FMT)];
    __shared__ int meta[2];
    const uint32_t * grid = stage_grid<FMT>(grid_lds);
    const int a = blockIdx.y, e = ids[a];
    if (e < 0 || int64_t(e) * b0.rows >= b0.rows_total) return;   // skipped assignment, or an id outside the bank
    int a1;
    const int cnt = pair_up(ids, A, a, e, mode, meta, a1);
    if (cnt == 0) return;
    constexpr int RW = 64 / LPR, kTile = NJ * NW * RW;
    const int S = b0.cols / 32, sl = (threadIdx.x & 63) % LPR, row0 = blockIdx.x * kTile, rows = b0.rows;
    const int s_end = (a % slots) < topk ? S : shared_cols / 32;   // the shared expert's input row may be narrower
    Tile tile[NB];
    tile[0] = tile_of<FMT>(b0, e, row0);
    if constexpr (NB == 2) tile[1] = tile_of<FMT>(b1, e, row0);
    auto store = [&](int a2, int nb, int r, float v) {
        if (row0 + r >= rows) return;
        const int64_t o = int64_t(a2) * rows + row0 + r;
        void * y = nb ? y1 : y0;
        if (ytype == TQMOE_F32) static_cast<float *>(y)[o] = v; else static_cast<uint16_t *>(y)[o] = float_to_bf16_bits(v);
    };
    if (cnt == 2) {
        const int xrow[2] = {a / xdiv, a1 / xdiv};
        ActBlock x[2][M];
        load_x<M, 2>(image, xrow, S, s_end, LPR, sl, x);
        block_rows<FMT, LPR, M, NB, 2, NJ, NW>(tile, S, rows - row0, x, grid, [&](int nb, int nt, int r, float v) { store(nt ? a1 : a, nb, r, v); });
    } else {
        const int xrow[1] = {a / xdiv};
        ActBlock x[1][M];
        load_x<M, 1>(image, xrow, S, s_end, LPR, sl, x);
        block_rows<FMT, LPR, M, NB, 1, NJ, NW>(tile, S, rows - row0, x, grid, [&](int nb, int, int r, float v) { store(a, nb, r, v); });
    }
}

// ------------------------------------------------------------------------- fused gate + up + SwiGLU (layer path)
// grid (ff / 32, n * slots), NW waves: one block makes one 32-value sub-block of act = silu(gate x) * (up x) for its
// assignment (and the paired one) and writes it straight into the activation image the down product reads. ids:
// [n][slots] expert of every (token, slot); slots past topk hold the shared expert, which only has shared_ff rows.
template <uint32_t FMT, int LPR, int M, int NW>
__global__ __launch_bounds__(NW * 64) void gateup_k(BankView bg, BankView bu, const uint8_t * __restrict__ ximage, uint8_t * __restrict__ aimage,
                                                    const int * __restrict__ ids, int A, int slots, int topk, int shared_ff, int mode, Glu glu) {
    constexpr int RW = 64 / LPR, NJ = 32 / (NW * RW);
    static_assert(NJ >= 1 && NJ * NW * RW == 32, "a block makes exactly 32 rows");
    __shared__ __attribute__((aligned(8))) uint32_t grid_lds[lattice_dwords(FMT)];
    __shared__ int meta[2];
    __shared__ float gl[2][32], ul[2][32];
    __shared__ int ql[2][32];
    const uint32_t * grid = stage_grid<FMT>(grid_lds);
    const int a = blockIdx.y, e = ids[a], row0 = blockIdx.x * 32;
    if (e < 0 || int64_t(e) * bg.rows >= bg.rows_total || row0 >= ((a % slots) < topk ? bg.rows : shared_ff)) return;
    int a1;
    const int cnt = pair_up(ids, A, a, e, mode, meta, a1);
    if (cnt == 0) return;
    const int S = bg.cols / 32, SA = bg.rows / 32, sl = (threadIdx.x & 63) % LPR;
    const Tile tile[2] = {tile_of<FMT>(bg, e, row0), tile_of<FMT>(bu, e, row0)};
    if (cnt == 2) {
        const int xrow[2] = {a / slots, a1 / slots};
        ActBlock x[2][M];
        load_x<M, 2>(ximage, xrow, S, S, LPR, sl, x);
        block_rows<FMT, LPR, M, 2, 2, NJ, NW>(tile, S, 32, x, grid, [&](int nb, int nt, int r, float v) { (nb ? ul : gl)[nt][r] = v; });
    } else {
        const int xrow[1] = {a / slots};
        ActBlock x[1][M];
        load_x<M, 1>(ximage, xrow, S, S, LPR, sl, x);
        block_rows<FMT, LPR, M, 2, 1, NJ, NW>(tile, S, 32, x, grid, [&](int nb, int, int r, float v) { (nb ? ul : gl)[0][r] = v; });
    }
    __syncthreads();
    // silu(g) * u of the 32 rows -> the activation image sub-block of each assignment: 32 lanes per assignment in wave 0
    const int tid = threadIdx.x, which = tid >> 5, i = tid & 31;
    if (tid < 64) {                                                 // the whole wave: the lane exchanges need every lane
        const bool live = which < cnt;
        float g = live ? gl[which][i] : 0.f, u = live ? ul[which][i] : 0.f;
        glu_clamp_inputs(glu, g, u);
        quantise_block_lanes(glu_clamp_silu(glu, g / (1.f + expf(-g))) * u, i, live, ql[which], aimage + int64_t(which ? a1 : a) * SA * kImageSubBytes, SA, blockIdx.x);
    }
}

// --------------------------------------------------------------------------------------------------- launchers
constexpr int kMatvecNJ = 4, kMatvecNW = 4;   // plain products: 4 row steps of 4 waves, 16 * (64 / LPR) rows per block
constexpr int kGateupNW = 8;                   // gate/up: 8 waves share the block's 32 + 32 rows

template <uint32_t FMT, int LPR, int M> void launch_one_matvec(int nb, const MatvecArgs & k, hipStream_t s) {
    constexpr int kTile = kMatvecNJ * kMatvecNW * (64 / LPR);
    const dim3 grid(unsigned((k.b0.rows + kTile - 1) / kTile), unsigned(k.A));
    if (nb == 2) matvec_k<FMT, LPR, M, 2, kMatvecNJ, kMatvecNW><<<grid, kMatvecNW * 64, 0, s>>>(k.b0, k.b1, k.image, k.y0, k.y1, k.ytype, k.ids, k.A, k.xdiv, k.mode, k.slots, k.topk, k.shared_cols);
    else matvec_k<FMT, LPR, M, 1, kMatvecNJ, kMatvecNW><<<grid, kMatvecNW * 64, 0, s>>>(k.b0, k.b1, k.image, k.y0, k.y1, k.ytype, k.ids, k.A, k.xdiv, k.mode, k.slots, k.topk, k.shared_cols);
}
template <uint32_t FMT, int LPR, int M> void launch_one_gateup(const GateupArgs & k, hipStream_t s) {
    const dim3 grid(unsigned(k.bg.rows / 32), unsigned(k.A));
    // as many waves as divide the block's 32 rows: 8 for 8 lanes or more per row
    constexpr int NW = 32 / (64 / LPR) >= kGateupNW ? kGateupNW : 32 / (64 / LPR);
    gateup_k<FMT, LPR, M, NW><<<grid, NW * 64, 0, s>>>(k.bg, k.bu, k.ximage, k.aimage, k.ids, k.A, k.slots, k.topk, k.shared_ff, k.mode, k.glu);
}

// the (lanes per row, sub-blocks per lane) pairs split_for() can return
#define TQMOE_FOR_SPLITS(X) X(64, 1) X(64, 2) X(64, 3) X(64, 4) X(32, 1) X(32, 3) X(16, 1) X(16, 3) X(8, 1) X(8, 3)

}  // namespace

template <uint32_t FMT> void DecodeLaunch<FMT>::matvec(Split sp, int nb, const MatvecArgs & k, hipStream_t s) {
#define X(L, MM) if (sp.lpr == L && sp.m == MM) return launch_one_matvec<FMT, L, MM>(nb, k, s);
    TQMOE_FOR_SPLITS(X)
#undef X
}
template <uint32_t FMT> void DecodeLaunch<FMT>::gateup(Split sp, const GateupArgs & k, hipStream_t s) {
#define X(L, MM) if (sp.lpr == L && sp.m == MM) return launch_one_gateup<FMT, L, MM>(k, s);
    TQMOE_FOR_SPLITS(X)
#undef X
}

}  // namespace tqmoe

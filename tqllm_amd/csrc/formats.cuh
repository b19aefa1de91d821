// Bank formats: device layout arithmetic and the per-sub-block decode shared by the loader, the fp32 dequantiser and
// the product kernels. A sub-block is 32 consecutive weights of a row; S = cols / 32 sub-blocks per row.
#pragma once
#include "common.cuh"
#include "iq3s_lattice.h"
#include "iq3xxs_lattice.h"
#include "iq2s_lattice.h"
#include "iq2xxs_lattice.h"
#include "iq2xs_lattice.h"
#include "iq1s_lattice.h"

namespace tqmoe {

// code bytes per sub-block
__host__ __device__ constexpr int code_bytes_per_sub(uint32_t type) {
    return type == TQMOE_IQ3_S || type == TQMOE_IQ3_XXS || type == TQMOE_IQ2_S || type == TQMOE_IQ2_XS || type == TQMOE_Q3_K ? 12
         : type == TQMOE_IQ2_XXS || type == TQMOE_Q2_K || type == TQMOE_IQ1_S ? 8 : type == TQMOE_Q8_0 ? 32 : type == TQMOE_Q6_K ? 24 : 16;
}
// aux record bytes per 256 weights (NVFP4G keeps bytes per 16 weights instead: see aux_row_bytes; IQ4_NL, Q4_0 and Q8_0
// hold the eight fp16 scales of their 32-weight blocks)
// Q5_K: the Q4_K header and the eight sub-blocks' high-bit words; Q6_K and Q3_K: sixteen int8 scales, d, padding;
// Q2_K: sixteen (scale | min << 4) bytes, d, dmin, padding
__host__ __device__ constexpr int aux_record_bytes(uint32_t type) { return type == TQMOE_IQ4_XS ? 8 : type == TQMOE_Q5_K ? 48 : type == TQMOE_Q6_K || type == TQMOE_Q3_K || type == TQMOE_Q2_K ? 32 : 16; }
__host__ __device__ constexpr int64_t code_row_bytes(uint32_t type, int cols) { return int64_t(cols / 32) * code_bytes_per_sub(type); }
__host__ __device__ constexpr int64_t aux_row_bytes(uint32_t type, int cols) {
    return type == TQMOE_NVFP4G ? int64_t(cols / 16) : int64_t(cols / 256) * aux_record_bytes(type);
}
// NVFP4G: offset of the per-row fp32 globals inside the aux plane
__host__ __device__ constexpr int64_t nvfp4_global_offset(int64_t rows_total, int cols) { return (rows_total * (cols / 16) + 15) / 16 * 16; }

// IQ4_XS banks are stored tile-major: 32 consecutive rows form a tile, and inside a tile the codes of sub-block s of
// all 32 rows are contiguous (512 B), as are the 32 records of a super-block (256 B). A wave then reads whole tiles with
// fully coalesced loads whichever lane owns which row. rows of an expert must be a multiple of 32.
__host__ __device__ constexpr int64_t iq4xs_code_offset(int64_t row, int S, int s) { return (((row >> 5) * S + s) * 32 + (row & 31)) * 16; }
__host__ __device__ constexpr int64_t iq4xs_aux_offset(int64_t row, int S, int sb) { return (((row >> 5) * (S >> 3) + sb) * 32 + (row & 31)) * 8; }

// IQ4_NL / IQ4_XS value table {-127,-104,-83,-65,-49,-35,-22,-10,1,13,25,38,53,69,89,113} as four little-endian dwords
constexpr uint32_t kIq4T0 = 0xBFAD9881u, kIq4T1 = 0xF6EADDCFu, kIq4T2 = 0x26190D01u, kIq4T3 = 0x71594535u;
// 2 * E2M1 {0,.5,1,1.5,2,3,4,6, -0,-.5,-1,-1.5,-2,-3,-4,-6} = {0,1,2,3,4,6,8,12, 0,-1,-2,-3,-4,-6,-8,-12}
constexpr uint32_t kFp4T0 = 0x03020100u, kFp4T1 = 0x0C080604u, kFp4T2 = 0xFDFEFF00u, kFp4T3 = 0xF4F8FAFCu;

// 8 four-bit codes of one dword -> int8 table values: lo = the four low nibbles, hi = the four high nibbles
template <uint32_t T0, uint32_t T1, uint32_t T2, uint32_t T3>
__device__ __forceinline__ void lookup16(uint32_t c, uint32_t & lo, uint32_t & hi) {
    // v_perm_b32 picks from an 8-byte pool, so: both halves of the table by the low three index bits, then a third
    // pick between the two results by index bit 3 (selector byte = position + 4 * bit3)
    const uint32_t i_lo = c & 0x07070707u, i_hi = (c >> 4) & 0x07070707u;
    const uint32_t a_lo = __builtin_amdgcn_perm(T1, T0, i_lo), b_lo = __builtin_amdgcn_perm(T3, T2, i_lo);
    const uint32_t a_hi = __builtin_amdgcn_perm(T1, T0, i_hi), b_hi = __builtin_amdgcn_perm(T3, T2, i_hi);
    lo = __builtin_amdgcn_perm(b_lo, a_lo, ((c >> 1) & 0x04040404u) | 0x03020100u);
    hi = __builtin_amdgcn_perm(b_hi, a_hi, ((c >> 5) & 0x04040404u) | 0x03020100u);
}
__device__ __forceinline__ void nibbles(uint32_t c, uint32_t & lo, uint32_t & hi) { lo = c & 0x0F0F0F0Fu; hi = (c >> 4) & 0x0F0F0F0Fu; }

// IQ3_S lattice points in the classic form (byte j = magnitude of weight j)
struct Iq3sGrid { uint32_t v[512]; };
constexpr Iq3sGrid make_iq3s_grid() {
    constexpr uint16_t codes[512] = {TQMOE_IQ3S_LATTICE12};
    Iq3sGrid g{};
    for (int i = 0; i < 512; ++i) {
        const uint32_t c = codes[i];
        g.v[i] = (2u * (c & 7u) + 1u) | ((2u * ((c >> 3) & 7u) + 1u) << 8) | ((2u * ((c >> 6) & 7u) + 1u) << 16) | ((2u * ((c >> 9) & 7u) + 1u) << 24);
    }
    return g;
}
__device__ const Iq3sGrid d_iq3s_grid = make_iq3s_grid();

// IQ3_XXS lattice points in the classic form
struct Iq3xxsGrid { uint32_t v[256]; };
constexpr uint32_t iq3xxs_level(uint32_t l) { return l < 7u ? 8u * l + 4u : 62u; }
constexpr Iq3xxsGrid make_iq3xxs_grid() {
    constexpr uint16_t codes[256] = {TQMOE_IQ3XXS_LATTICE12};
    Iq3xxsGrid g{};
    for (int i = 0; i < 256; ++i) {
        const uint32_t c = codes[i];
        g.v[i] = iq3xxs_level(c & 7u) | (iq3xxs_level((c >> 3) & 7u) << 8) | (iq3xxs_level((c >> 6) & 7u) << 16) | (iq3xxs_level((c >> 9) & 7u) << 24);
    }
    return g;
}
__device__ const Iq3xxsGrid d_iq3xxs_grid = make_iq3xxs_grid();
// IQ2_S / IQ2_XS / IQ2_XXS lattice points: two dwords per point (magnitudes of weights 0..3, 4..7 of the group of eight)
template <int N> struct Iq2Grid { uint32_t v[2 * N]; };
template <int N> constexpr Iq2Grid<N> make_iq2_grid(const uint16_t (&codes)[N]) {
    constexpr uint32_t level[4] = {8, 25, 43, 0};
    Iq2Grid<N> g{};
    for (int i = 0; i < N; ++i)
        for (int h = 0; h < 2; ++h) {
            uint32_t w = 0;
            for (int j = 0; j < 4; ++j) w |= level[(codes[i] >> (2 * (4 * h + j))) & 3u] << (8 * j);
            g.v[2 * i + h] = w;
        }
    return g;
}
constexpr uint16_t kIq2sCodes[1024] = {TQMOE_IQ2S_LATTICE16};
constexpr uint16_t kIq2xsCodes[512] = {TQMOE_IQ2XS_LATTICE16};
constexpr uint16_t kIq2xxsCodes[256] = {TQMOE_IQ2XXS_LATTICE16};
__device__ const Iq2Grid<1024> d_iq2s_grid = make_iq2_grid(kIq2sCodes);
__device__ const Iq2Grid<512> d_iq2xs_grid = make_iq2_grid(kIq2xsCodes);
__device__ const Iq2Grid<256> d_iq2xxs_grid = make_iq2_grid(kIq2xxsCodes);
// IQ1_S lattice points: two dwords per point, int8 values from {-1, 0, 1}
constexpr Iq2Grid<2048> make_iq1s_grid() {
    constexpr uint16_t codes[2048] = {TQMOE_IQ1S_LATTICE16};
    constexpr uint32_t value[4] = {0x00, 0x01, 0xFF, 0};
    Iq2Grid<2048> g{};
    for (int i = 0; i < 2048; ++i)
        for (int h = 0; h < 2; ++h) {
            uint32_t w = 0;
            for (int j = 0; j < 4; ++j) w |= value[(codes[i] >> (2 * (4 * h + j))) & 3u] << (8 * j);
            g.v[2 * i + h] = w;
        }
    return g;
}
__device__ const Iq2Grid<2048> d_iq1s_grid = make_iq1s_grid();
// dwords of a format's lattice as the kernels stage it in LDS (1: the format has none)
__host__ __device__ constexpr int lattice_dwords(uint32_t type) {
    return type == TQMOE_IQ3_S ? 512 : type == TQMOE_IQ3_XXS ? 256 : type == TQMOE_IQ2_S ? 2048 : type == TQMOE_IQ2_XS ? 1024 : type == TQMOE_IQ2_XXS ? 512 : type == TQMOE_IQ1_S ? 4096 : 1;
}
// lattice index of group l of an IQ2_S sub-block: its low byte and two bits of the sub-block's qh byte
__device__ __forceinline__ uint32_t iq2s_index(uint32_t low4, uint32_t qh, int l) { return ((low4 >> (8 * l)) & 0xFFu) | ((qh << (8 - 2 * l)) & 0x300u); }

// the eight sign bits of a group of eight weights from its seven stored ones: the eighth makes their count even
__device__ __forceinline__ uint32_t signs8(uint32_t i7) { return i7 | ((uint32_t(__popc(i7)) & 1u) << 7); }
__device__ __forceinline__ uint32_t iq3xxs_signs(uint32_t word, int l) { return signs8((word >> (7 * l)) & 127u); }
// the magnitudes g of four weights with the signs of four bits applied: negate the selected bytes, (g ^ m) + bits with m
// the byte masks 0xFF of the set bits; no carry leaves a byte
__device__ __forceinline__ uint32_t apply_signs4(uint32_t g, uint32_t bits4);

// E4M3 byte -> float: (1 + m/8) 2^(e-7), subnormal m/8 2^-6, 0x7F / 0xFF NaN
__device__ __forceinline__ float e4m3_to_float(uint32_t b) {
    const int e = (b >> 3) & 15, m = b & 7;
    float v;
    if (e == 15 && m == 7) v = __uint_as_float(0x7FC00000u);
    else if (e == 0) v = float(m) * 0.001953125f;                          // m * 2^-9
    else v = __uint_as_float(uint32_t(e + 120) << 23 | uint32_t(m) << 20);  // (1 + m/8) * 2^(e - 7)
    return (b & 0x80u) ? -v : v;
}

// the same through the fp16 conversion: the seven low bits moved to fp16's exponent and mantissa fields are the value
// times 2^-8, subnormals included (one conversion and one multiply); the NaN codes are kept
__device__ __forceinline__ float e4m3_to_float_fast(uint32_t b) {
    const float v = half_bits_to_float(uint16_t(((b & 0x80u) << 8) | ((b & 0x7Fu) << 7))) * 256.f;
    return (b & 0x7Fu) == 0x7Fu ? __uint_as_float(0x7FC00000u) : v;
}

// four bits -> the low bit of four bytes
__device__ __forceinline__ uint32_t spread4(uint32_t bits) { return ((bits & 15u) * 0x00204081u) & 0x01010101u; }
// eight bits (four 2-bit fields) -> the low two bits of four bytes
__device__ __forceinline__ uint32_t spread2x4(uint32_t x) { x &= 0xFFu; return (x | x << 6 | x << 12 | x << 18) & 0x03030303u; }
// bytes q in [0, 63] -> int8 bytes q - 32
__device__ __forceinline__ uint32_t minus32(uint32_t v) { return ((v | 0x80808080u) - 0x20202020u) ^ 0x80808080u; }
// bytes q in [0, 127] -> int8 bytes q - K
template <uint32_t K> __device__ __forceinline__ uint32_t minus_k(uint32_t v) { return ((v | 0x80808080u) - K * 0x01010101u) ^ 0x80808080u; }
__device__ __forceinline__ uint32_t apply_signs4(uint32_t g, uint32_t bits4) {
    const uint32_t bits = spread4(bits4), m = (bits << 8) - bits;
    return (g ^ m) + bits;
}

// Q4_K: 6-bit (scale, min) of sub-block j from the 12-byte field held as three dwords
__device__ __forceinline__ void q4k_scale_min(const uint32_t (&q)[3], int j, int & sc, int & mn) {
    auto byte = [&](int i) { return (q[i >> 2] >> (8 * (i & 3))) & 0xFFu; };
    if (j < 4) { sc = byte(j) & 63; mn = byte(j + 4) & 63; }
    else { sc = (byte(j + 4) & 15) | ((byte(j - 4) >> 6) << 4); mn = (byte(j + 4) >> 4) | ((byte(j) >> 6) << 4); }
}

// the same without a branch or an indexed read, for a sub-block number that is only known at run time: bytes j % 4 of the
// three dwords are all that either case reads (a branch here splits the caller's loop body into blocks, and work that
// the compiler then moves across them stays in registers for the whole body)
__device__ __forceinline__ void q4k_scale_min_flat(uint32_t q0, uint32_t q1, uint32_t q2, int j, int & sc, int & mn) {
    const int sh = 8 * (j & 3);
    const uint32_t a = (q0 >> sh) & 0xFFu, b = (q1 >> sh) & 0xFFu, c = (q2 >> sh) & 0xFFu;
    const bool low = j < 4;
    sc = int(low ? a & 63u : (c & 15u) | ((a >> 6) << 4));
    mn = int(low ? b & 63u : (c >> 4) | ((b >> 6) << 4));
}

// IQ4_XS: the 8-byte record of a 256-weight super-block as the device holds it. GGUF's (d, scales_h, scales_l[4]) is the
// same 64 bits arranged for extraction in one instruction each: the eight 6-bit scales are stored minus 32 as signed
// fields (what the decoder multiplies by), five in x at bits 6 ib, three in y at bits 14 + 6 (ib - 5); the fp16 d sits in
// the 16 bits between them (x bits 30..31, y bits 0..13), which one alignbit brings to the low half.
__host__ __device__ inline uint2 iq4xs_pack_rec(uint32_t d_bits, uint32_t scales_h, uint32_t scales_l) {
    uint32_t x = 0, y = 0;
    for (int ib = 0; ib < 8; ++ib) {
        const uint32_t ls = ((scales_l >> (4 * ib)) & 15u) | (((scales_h >> (2 * ib)) & 3u) << 4);
        const uint32_t f = (ls - 32u) & 63u;
        if (ib < 5) x |= f << (6 * ib); else y |= f << (14 + 6 * (ib - 5));
    }
    x |= (d_bits & 3u) << 30;
    y |= (d_bits >> 2) & 0x3FFFu;
    return uint2{x, y};
}
// scale of sub-block ib minus 32, in [-32, 31]
__device__ __forceinline__ int iq4xs_lsm32(uint2 rec, int ib) {
    return ib < 5 ? __builtin_amdgcn_sbfe(int(rec.x), 6 * ib, 6) : __builtin_amdgcn_sbfe(int(rec.y), 14 + 6 * (ib - 5), 6);
}
__device__ __forceinline__ int iq4xs_ls(uint2 rec, int ib) { return iq4xs_lsm32(rec, ib) + 32; }
__device__ __forceinline__ uint16_t iq4xs_d_bits(uint2 rec) { return uint16_t(__builtin_amdgcn_alignbit(rec.y, rec.x, 30) & 0xFFFFu); }

}  // namespace tqmoe

// CPU oracle for the mixture-of-experts layer: TEST INFRASTRUCTURE ONLY (see tqmoe_oracle.h for what each function
// follows in the reference and how it is pinned). Nothing in the product library links or loads this file.
#include "tqmoe_oracle.h"
#include "iq3s_lattice.h"
#include "iq3xxs_lattice.h"
#include "iq2s_lattice.h"
#include "iq2xxs_lattice.h"
#include "iq2xs_lattice.h"
#include "iq1s_lattice.h"

#include <immintrin.h>

#include <algorithm>
#include <atomic>
#include <chrono>
#include <cmath>
#include <cstring>
#include <functional>
#include <limits>
#include <mutex>
#include <numeric>
#include <thread>
#include <vector>

namespace {

const int8_t kIq4Values[16] = {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113};
const float kE2M1[16] = {0.f, 0.5f, 1.f, 1.5f, 2.f, 3.f, 4.f, 6.f, -0.f, -0.5f, -1.f, -1.5f, -2.f, -3.f, -4.f, -6.f};

inline uint32_t f2u(float f) { uint32_t u; std::memcpy(&u, &f, 4); return u; }
inline float u2f(uint32_t u) { float f; std::memcpy(&f, &u, 4); return f; }
inline uint16_t rd16(const uint8_t * p) { uint16_t v; std::memcpy(&v, p, 2); return v; }

}  // namespace

// ---------------------------------------------------------------------------------------------- conversions
// src/formats/weight/dequant.cpp:32-54: IEEE binary16 -> binary32, subnormals, inf and NaN payload kept.
float tqo_half_to_float(uint16_t h) {
    const uint32_t sign = uint32_t(h >> 15) << 31;
    const int e = (h >> 10) & 31;
    uint32_t m = h & 1023u;
    if (e == 31) return u2f(sign | 0x7F800000u | (m << 13));
    if (e) return u2f(sign | uint32_t(e + 112) << 23 | (m << 13));
    if (!m) return u2f(sign);
    int shift = 0;  // normalise the subnormal: value = m * 2^-24
    while (!(m & 1024u)) { m <<= 1; ++shift; }
    return u2f(sign | uint32_t(113 - shift) << 23 | ((m & 1023u) << 13));
}

// src/formats/weight/dequant.cpp:12-30: binary32 -> binary16, round to nearest even, overflow to inf.
uint16_t tqo_float_to_half(float f) {
    const uint32_t x = f2u(f), a = x & 0x7FFFFFFFu;
    const uint16_t sign = uint16_t((x >> 16) & 0x8000u);
    if (a > 0x7F800000u) return uint16_t(sign | 0x7E00u);
    if (a == 0x7F800000u) return uint16_t(sign | 0x7C00u);
    // work on the exact value: a = mant * 2^(e - 150)
    const int e = int(a >> 23);
    if (e < 102) return sign;  // below half the smallest subnormal (2^-25): zero; e == 102 may round up
    uint32_t mant = (a & 0x7FFFFFu) | (e ? 0x800000u : 0u);
    // target unit: 2^-24 for subnormal halves (e <= 112), else 2^(e - 127 - 10)
    const int drop = e <= 112 ? 126 - e : 13;  // bits of mant below the target unit
    uint32_t q = drop >= 32 ? 0 : mant >> drop;
    const uint32_t rest = mant & ((1u << drop) - 1u), half = 1u << (drop - 1);
    if (rest > half || (rest == half && (q & 1u))) ++q;
    if (e <= 112) return uint16_t(sign | q);  // q == 1024 lands on the smallest normal by construction
    // q in [1024, 2048]; exponent field e - 112
    uint32_t bits = (uint32_t(e - 112) << 10) + (q - 1024u);
    if (bits >= 0x7C00u) bits = 0x7C00u;
    return uint16_t(sign | bits);
}

float tqo_bf16_to_float(uint16_t h) { return u2f(uint32_t(h) << 16); }
uint16_t tqo_float_to_bf16(float f) {
    const uint32_t x = f2u(f);
    if ((x & 0x7FFFFFFFu) > 0x7F800000u) return uint16_t((x >> 16) | 0x40u);
    return uint16_t((x + 0x7FFFu + ((x >> 16) & 1u)) >> 16);
}

// src/formats/weight/dequant.cpp:387-391
float tqo_e4m3_to_float(uint8_t b) {
    const int e = (b >> 3) & 15, m = b & 7;
    float v;
    if (e == 15 && m == 7) v = std::numeric_limits<float>::quiet_NaN();
    else if (e == 0) v = std::ldexp(float(m), -9);
    else v = std::ldexp(float(8 + m), e - 10);
    return (b & 0x80) ? -v : v;
}

uint8_t tqo_float_to_e4m3(float f) {
    const uint8_t sign = (f2u(f) >> 31) ? 0x80 : 0;
    const float a = std::fabs(f);
    if (a != a) return uint8_t(sign | 0x7F);
    if (a >= 448.f) return uint8_t(sign | 0x7E);
    if (a < 0.015625f) {  // below 2^-6: subnormal step 2^-9
        const int m = int(std::nearbyint(std::ldexp(a, 9)));
        return uint8_t(sign | m);  // m == 8 is the code of 2^-6
    }
    int ex;
    const float fr = std::frexp(a, &ex);            // a = fr * 2^ex, fr in [0.5, 1)
    int m = int(std::nearbyint(std::ldexp(fr, 4)));  // 8..16 in units of 2^(ex - 4)
    int e = ex - 1 + 7;
    if (m == 16) { m = 8; ++e; }
    int code = (e << 3) | (m - 8);
    if (code > 0x7E) code = 0x7E;
    return uint8_t(sign | code);
}

// ------------------------------------------------------------------------------------------------- decoding
int tqo_block_layout(uint32_t type, int * elems, int * bytes) {
    int e = 0, b = 0;
    switch (type) {  // src/core/gguf.cpp:136-152
        case TQO_Q4_K: e = 256; b = 144; break;
        case TQO_Q5_K: e = 256; b = 176; break;
        case TQO_Q6_K: e = 256; b = 210; break;
        case TQO_IQ4_NL: e = 32; b = 18; break;
        case TQO_Q8_0: e = 32; b = 34; break;
        case TQO_IQ3_S: e = 256; b = 110; break;
        case TQO_IQ3_XXS: e = 256; b = 98; break;
        case TQO_IQ2_S: e = 256; b = 82; break;
        case TQO_IQ2_XXS: e = 256; b = 66; break;
        case TQO_IQ2_XS: e = 256; b = 74; break;
        case TQO_Q3_K: e = 256; b = 110; break;
        case TQO_Q4_0: e = 32; b = 18; break;
        case TQO_Q2_K: e = 256; b = 84; break;
        case TQO_IQ1_S: e = 256; b = 50; break;
        case TQO_IQ4_XS: e = 256; b = 136; break;
        case TQO_NVFP4G: e = 128; b = 76; break;
        default: return 0;
    }
    if (elems) *elems = e;
    if (bytes) *bytes = b;
    return 1;
}

namespace {

// 6-bit (scale, min) pair j of a Q4_K block's 12-byte field, src/formats/weight/dequant.cpp:56-64
inline void q4k_scale_min(const uint8_t * q, int j, int & sc, int & mn) {
    if (j < 4) { sc = q[j] & 63; mn = q[j + 4] & 63; }
    else { sc = (q[j + 4] & 15) | ((q[j - 4] >> 6) << 4); mn = (q[j + 4] >> 4) | ((q[j] >> 6) << 4); }
}

void decode_q4k(const uint8_t * b, float * y) {
    const float d = tqo_half_to_float(rd16(b)), dmin = tqo_half_to_float(rd16(b + 2));
    for (int c = 0; c < 4; ++c) {
        int s1, m1, s2, m2;
        q4k_scale_min(b + 4, 2 * c, s1, m1);
        q4k_scale_min(b + 4, 2 * c + 1, s2, m2);
        // evaluation order of the reference: (d * sc) * code - (dmin * m)
        const float d1 = d * float(s1), o1 = dmin * float(m1), d2 = d * float(s2), o2 = dmin * float(m2);
        const uint8_t * q = b + 16 + 32 * c;
        for (int l = 0; l < 32; ++l) {
            y[64 * c + l] = d1 * float(q[l] & 15) - o1;
            y[64 * c + 32 + l] = d2 * float(q[l] >> 4) - o2;
        }
    }
}

void decode_q5k(const uint8_t * b, float * y) {  // src/formats/weight/dequant.cpp:102-116: (d * sc) * v - dmin * m
    const float d = tqo_half_to_float(rd16(b)), dmin = tqo_half_to_float(rd16(b + 2));
    const uint8_t * qh = b + 16, * q = b + 48;
    for (int j = 0; j < 8; ++j) {
        int sc, mn;
        q4k_scale_min(b + 4, j, sc, mn);
        for (int l = 0; l < 32; ++l) {
            const int v = ((j & 1) ? q[32 * (j / 2) + l] >> 4 : q[32 * (j / 2) + l] & 15) + ((qh[l] >> j) & 1) * 16;
            y[32 * j + l] = d * float(sc) * float(v) - dmin * float(mn);
        }
    }
}

void decode_q6k(const uint8_t * b, float * y) {  // src/formats/weight/dequant.cpp:194-208: (d * sc) * (q - 32)
    const uint8_t * ql = b, * qh = b + 128;
    const int8_t * sc = reinterpret_cast<const int8_t *>(b + 192);
    const float d = tqo_half_to_float(rd16(b + 208));
    for (int n = 0; n < 2; ++n, y += 128, ql += 64, qh += 32, sc += 8)
        for (int l = 0; l < 32; ++l) {
            const int is = l / 16;
            y[l] = d * float(sc[is]) * float(((ql[l] & 15) | (((qh[l] >> 0) & 3) << 4)) - 32);
            y[l + 32] = d * float(sc[is + 2]) * float(((ql[l + 32] & 15) | (((qh[l] >> 2) & 3) << 4)) - 32);
            y[l + 64] = d * float(sc[is + 4]) * float(((ql[l] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32);
            y[l + 96] = d * float(sc[is + 6]) * float(((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32);
        }
}

inline int iq4xs_subscale(const uint8_t * b, int ib) {  // 6-bit scale of sub-block ib, before the -32 offset
    const uint16_t sh = rd16(b + 2);
    return ((b[4 + ib / 2] >> (4 * (ib & 1))) & 15) | (((sh >> (2 * ib)) & 3) << 4);
}

void decode_iq4xs(const uint8_t * b, float * y) {
    const float d = tqo_half_to_float(rd16(b));
    for (int ib = 0; ib < 8; ++ib) {
        const float dl = d * float(iq4xs_subscale(b, ib) - 32);
        const uint8_t * q = b + 8 + 16 * ib;
        for (int j = 0; j < 16; ++j) {
            y[32 * ib + j] = dl * float(kIq4Values[q[j] & 15]);
            y[32 * ib + 16 + j] = dl * float(kIq4Values[q[j] >> 4]);
        }
    }
}

void decode_iq4nl(const uint8_t * b, float * y) {
    const float d = tqo_half_to_float(rd16(b));
    for (int j = 0; j < 16; ++j) {
        y[j] = d * float(kIq4Values[b[2 + j] & 15]);
        y[16 + j] = d * float(kIq4Values[b[2 + j] >> 4]);
    }
}

void decode_iq3xxs(const uint8_t * b, float * y) {  // src/formats/weight/dequant.cpp:157-174
    const float d = tqo_half_to_float(rd16(b));
    const uint8_t * qs = b + 2;
    for (int ib = 0; ib < 8; ++ib) {
        uint32_t a;
        std::memcpy(&a, b + 66 + 4 * ib, 4);
        const float db = d * (0.5f + float(a >> 28)) * 0.5f;
        for (int l = 0; l < 4; ++l) {
            // seven stored sign bits for eight weights; the eighth makes the number of minus signs even
            const uint32_t i7 = (a >> (7 * l)) & 127u, sg = i7 | ((uint32_t(__builtin_popcount(i7)) & 1u) << 7);
            for (int h = 0; h < 2; ++h, y += 4) {
                const uint32_t g = tq_iq3xxs_point(qs[ib * 8 + 2 * l + h]);
                for (int j = 0; j < 4; ++j) y[j] = db * float((g >> (8 * j)) & 0xFFu) * (((sg >> (4 * h + j)) & 1u) ? -1.f : 1.f);
            }
        }
    }
}

void decode_iq2s(const uint8_t * b, float * y) {  // src/formats/weight/dequant.cpp:271-287
    const float d = tqo_half_to_float(rd16(b));
    const uint8_t * qs = b + 2, * signs = b + 34, * qh = b + 66, * sc = b + 74;
    for (int ib = 0; ib < 8; ++ib) {
        const float db[2] = {d * (0.5f + float(sc[ib] & 15)) * 0.25f, d * (0.5f + float(sc[ib] >> 4)) * 0.25f};
        for (int l = 0; l < 4; ++l) {
            const uint64_t g = tq_iq2s_point(qs[4 * ib + l] | ((qh[ib] << (8 - 2 * l)) & 0x300));
            for (int j = 0; j < 8; ++j)
                y[32 * ib + 8 * l + j] = db[l / 2] * float((g >> (8 * j)) & 0xFFu) * ((signs[4 * ib + l] >> j) & 1 ? -1.f : 1.f);
        }
    }
}

// the eight sign bits of a group of eight weights from a 7-bit field: the eighth makes the count of minus signs even
// (ksigns_iq2xs of the reference, src/formats/weight/ksigns_iq2xs.inc: entry i is i | parity(i) << 7)
inline uint32_t signs8(uint32_t i7) { return i7 | ((uint32_t(__builtin_popcount(i7)) & 1u) << 7); }

void decode_iq2xxs(const uint8_t * b, float * y) {  // src/formats/weight/dequant.cpp:233-249
    const float d = tqo_half_to_float(rd16(b));
    for (int ib = 0; ib < 8; ++ib) {
        uint32_t a[2];
        std::memcpy(a, b + 2 + 8 * ib, 8);
        const float db = d * (0.5f + float(a[1] >> 28)) * 0.25f;
        for (int l = 0; l < 4; ++l) {
            const uint64_t g = tq_iq2xxs_point((a[0] >> (8 * l)) & 0xFFu);
            const uint32_t sg = signs8((a[1] >> (7 * l)) & 127u);
            for (int j = 0; j < 8; ++j) y[32 * ib + 8 * l + j] = db * float((g >> (8 * j)) & 0xFFu) * (((sg >> j) & 1u) ? -1.f : 1.f);
        }
    }
}

void decode_iq2xs(const uint8_t * b, float * y) {  // src/formats/weight/dequant.cpp:252-268
    const float d = tqo_half_to_float(rd16(b));
    const uint8_t * sc = b + 66;
    for (int ib = 0; ib < 8; ++ib) {
        const float db[2] = {d * (0.5f + float(sc[ib] & 15)) * 0.25f, d * (0.5f + float(sc[ib] >> 4)) * 0.25f};
        for (int l = 0; l < 4; ++l) {
            const uint32_t q = rd16(b + 2 + 2 * (4 * ib + l));
            const uint64_t g = tq_iq2xs_point(q & 511u);
            const uint32_t sg = signs8(q >> 9);
            for (int j = 0; j < 8; ++j) y[32 * ib + 8 * l + j] = db[l / 2] * float((g >> (8 * j)) & 0xFFu) * (((sg >> j) & 1u) ? -1.f : 1.f);
        }
    }
}

void q3k_scales(const uint8_t * p, int8_t * sc) {  // src/formats/weight/dequant.cpp:66-76: 12 bytes -> 16 six-bit scales minus 32
    // scale i: low four bits in byte i % 8 (low nibble for i < 8, high for i >= 8), upper two bits in byte 8 + i % 4 at 2 (i / 4)
    for (int i = 0; i < 16; ++i) {
        const int lo = i < 8 ? p[i] & 15 : p[i - 8] >> 4;
        const int hi = (p[8 + (i & 3)] >> (2 * (i >> 2))) & 3;
        sc[i] = int8_t((lo | (hi << 4)) - 32);
    }
}

void decode_q3k(const uint8_t * b, float * y) {  // src/formats/weight/dequant.cpp:118-131: (d * sc) * q, q = two bits - (mask bit ? 0 : 4)
    int8_t sc[16];
    q3k_scales(b + 96, sc);
    const float d = tqo_half_to_float(rd16(b + 108));
    for (int e = 0; e < 256; ++e) {
        const int n = e / 128, j = (e % 128) / 32, w = e % 32;
        const int q = ((b[32 + 32 * n + w] >> (2 * j)) & 3) - (((b[w] >> (4 * n + j)) & 1) ? 0 : 4);
        y[e] = d * float(sc[8 * n + 2 * j + (w >= 16)]) * float(q);
    }
}

void decode_q2k(const uint8_t * b, float * y) {  // src/formats/weight/dequant.cpp:289-310: (d * scale) * q - dmin * min per 16 weights
    const float d = tqo_half_to_float(rd16(b + 80)), dmin = tqo_half_to_float(rd16(b + 82));
    for (int e = 0; e < 256; ++e) {
        const int n = e / 128, j = (e % 128) / 32, w = e % 32;
        const uint8_t sc = b[8 * n + 2 * j + (w >= 16)];
        const float dl = d * float(sc & 15), ml = dmin * float(sc >> 4);
        y[e] = dl * float((b[16 + 32 * n + w] >> (2 * j)) & 3) - ml;
    }
}

void decode_iq1s(const uint8_t * b, float * y) {  // src/formats/weight/dequant.cpp:311-326: (d * (2 s + 1)) * (value + delta)
    const float d = tqo_half_to_float(rd16(b));
    for (int ib = 0; ib < 8; ++ib) {
        const uint32_t qh = rd16(b + 34 + 2 * ib);
        const float dl = d * float(2 * ((qh >> 12) & 7) + 1), delta = (qh & 0x8000u) ? -0.125f : 0.125f;
        for (int l = 0; l < 4; ++l) {
            const uint64_t g = tq_iq1s_point(b[2 + 4 * ib + l] | (((qh >> (3 * l)) & 7u) << 8));
            for (int j = 0; j < 8; ++j) y[32 * ib + 8 * l + j] = dl * (float(int8_t((g >> (8 * j)) & 0xFFu)) + delta);
        }
    }
}

void decode_q4_0(const uint8_t * b, float * y) {  // src/formats/weight/dequant.cpp:480-491: (q - 8) * d
    const float d = tqo_half_to_float(rd16(b));
    for (int j = 0; j < 16; ++j) {
        y[j] = float(int(b[2 + j] & 15) - 8) * d;
        y[16 + j] = float(int(b[2 + j] >> 4) - 8) * d;
    }
}

void decode_q8_0(const uint8_t * b, float * y) {  // src/formats/weight/dequant.cpp:555-562
    const float d = tqo_half_to_float(rd16(b));
    for (int j = 0; j < 32; ++j) y[j] = d * float(int8_t(b[2 + j]));
}

void decode_iq3s(const uint8_t * b, float * y) {
    const float d = tqo_half_to_float(rd16(b));
    const uint8_t * qs = b + 2, * qh = b + 66, * signs = b + 74, * sc = b + 106;
    for (int ib = 0; ib < 8; ++ib) {
        const float db = d * float(1 + 2 * ((sc[ib / 2] >> (4 * (ib & 1))) & 15));
        for (int w = 0; w < 8; ++w) {
            const uint32_t g = tq_iq3s_point(qs[8 * ib + w] | (((qh[ib] >> w) & 1) << 8));
            const int sg = signs[4 * ib + w / 2] >> (4 * (w & 1));
            for (int j = 0; j < 4; ++j) {
                const float mag = db * float((g >> (8 * j)) & 255u);
                y[32 * ib + 4 * w + j] = ((sg >> j) & 1) ? mag * -1.f : mag * 1.f;
            }
        }
    }
}

void decode_nvfp4g(const uint8_t * b, float * y) {
    float g;
    std::memcpy(&g, b, 4);
    for (int grp = 0; grp < 8; ++grp) {
        const float d = tqo_e4m3_to_float(b[4 + grp]) * g;
        for (int i = 0; i < 8; ++i) {
            const uint8_t q = b[12 + 8 * grp + i];
            y[16 * grp + 2 * i] = kE2M1[q & 15] * d;
            y[16 * grp + 2 * i + 1] = kE2M1[q >> 4] * d;
        }
    }
}

}  // namespace

// NVFP4G with the weights as an fp8 matrix pipe takes them: e2m1 * E4M3 scale / 8 rounded to E4M3 (nearest even; the
// division keeps the largest product, 6 * 448 / 8 = 336, inside the format), 8 * the row's fp32 global applied to the rounded
// value (src/core/fp8_gemm.cuh:19-31 keeps scales outside the operand the same way)
int tqo_dequantize_nvfp4_widened(const void * src, float * dst, int64_t n) {
    if (n % 128) return -1;
    const uint8_t * b = static_cast<const uint8_t *>(src);
    for (int64_t blk = 0; blk < n / 128; ++blk, b += 76, dst += 128) {
        float g;
        std::memcpy(&g, b, 4);
        for (int grp = 0; grp < 8; ++grp) {
            const float sc = tqo_e4m3_to_float(b[4 + grp]);
            for (int i = 0; i < 8; ++i) {
                const uint8_t q = b[12 + 8 * grp + i];
                dst[16 * grp + 2 * i] = tqo_e4m3_to_float(tqo_float_to_e4m3(kE2M1[q & 15] * sc * 0.125f)) * (8.f * g);
                dst[16 * grp + 2 * i + 1] = tqo_e4m3_to_float(tqo_float_to_e4m3(kE2M1[q >> 4] * sc * 0.125f)) * (8.f * g);
            }
        }
    }
    return 0;
}

int tqo_dequantize(uint32_t type, const void * src, float * dst, int64_t n) {
    int elems, bytes;
    if (!tqo_block_layout(type, &elems, &bytes) || n < 0 || n % elems) return -1;
    const uint8_t * s = static_cast<const uint8_t *>(src);
    for (int64_t b = 0; b < n / elems; ++b, s += bytes, dst += elems) switch (type) {
        case TQO_Q4_K: decode_q4k(s, dst); break;
        case TQO_Q5_K: decode_q5k(s, dst); break;
        case TQO_Q6_K: decode_q6k(s, dst); break;
        case TQO_IQ4_XS: decode_iq4xs(s, dst); break;
        case TQO_IQ4_NL: decode_iq4nl(s, dst); break;
        case TQO_Q8_0: decode_q8_0(s, dst); break;
        case TQO_IQ3_S: decode_iq3s(s, dst); break;
        case TQO_IQ3_XXS: decode_iq3xxs(s, dst); break;
        case TQO_IQ2_S: decode_iq2s(s, dst); break;
        case TQO_IQ2_XXS: decode_iq2xxs(s, dst); break;
        case TQO_IQ2_XS: decode_iq2xs(s, dst); break;
        case TQO_Q3_K: decode_q3k(s, dst); break;
        case TQO_Q4_0: decode_q4_0(s, dst); break;
        case TQO_Q2_K: decode_q2k(s, dst); break;
        case TQO_IQ1_S: decode_iq1s(s, dst); break;
        case TQO_NVFP4G: decode_nvfp4g(s, dst); break;
    }
    return 0;
}

// ------------------------------------------------------------------------------------ encoders (own; unpinned)
namespace {

inline int nearest_iq4(float v) {  // index of the table value nearest to v, lower index on a tie
    int best = 0;
    float bd = std::fabs(v - float(kIq4Values[0]));
    for (int i = 1; i < 16; ++i) {
        const float dd = std::fabs(v - float(kIq4Values[i]));
        if (dd < bd) { bd = dd; best = i; }
    }
    return best;
}

// sub-block scale that puts the largest-magnitude value on table entry 0 (-127)
inline float iq4_block_scale(const float * x) {
    float amax = 0.f, vmax = 0.f;
    for (int i = 0; i < 32; ++i) if (std::fabs(x[i]) > amax) { amax = std::fabs(x[i]); vmax = x[i]; }
    return vmax / -127.f;
}

void encode_q8_0(const float * x, uint8_t * b) {  // d = amax / 127, q = rint(x / d)
    float amax = 0.f;
    for (int j = 0; j < 32; ++j) amax = std::max(amax, std::fabs(x[j]));
    const uint16_t hd = tqo_float_to_half(amax / 127.f);
    const float d = tqo_half_to_float(hd), inv = d != 0.f ? 1.f / d : 0.f;
    std::memcpy(b, &hd, 2);
    for (int j = 0; j < 32; ++j) b[2 + j] = uint8_t(int8_t(std::max(-127.f, std::min(127.f, std::nearbyint(x[j] * inv)))));
}

void encode_iq4nl(const float * x, uint8_t * b) {
    const uint16_t hd = tqo_float_to_half(iq4_block_scale(x));
    const float d = tqo_half_to_float(hd), inv = d != 0.f ? 1.f / d : 0.f;
    std::memcpy(b, &hd, 2);
    for (int j = 0; j < 16; ++j)
        b[2 + j] = uint8_t(nearest_iq4(x[j] * inv) | (nearest_iq4(x[16 + j] * inv) << 4));
}

void encode_iq4xs(const float * x, uint8_t * b) {
    float ds[8], big = 0.f;
    for (int ib = 0; ib < 8; ++ib) { ds[ib] = iq4_block_scale(x + 32 * ib); if (std::fabs(ds[ib]) > std::fabs(big)) big = ds[ib]; }
    const uint16_t hd = tqo_float_to_half(big / -32.f);  // the largest sub-scale sits on ls - 32 = -32
    const float d = tqo_half_to_float(hd);
    std::memset(b, 0, 136);
    std::memcpy(b, &hd, 2);
    uint16_t sh = 0;
    for (int ib = 0; ib < 8; ++ib) {
        int l = d != 0.f ? int(std::nearbyint(ds[ib] / d)) : 0;
        l = std::max(-32, std::min(31, l));
        const int ls = l + 32;
        b[4 + ib / 2] |= uint8_t((ls & 15) << (4 * (ib & 1)));
        sh |= uint16_t((ls >> 4) << (2 * ib));
        const float dl = d * float(l), inv = dl != 0.f ? 1.f / dl : 0.f;
        const float * v = x + 32 * ib;
        for (int j = 0; j < 16; ++j)
            b[8 + 16 * ib + j] = uint8_t(nearest_iq4(v[j] * inv) | (nearest_iq4(v[16 + j] * inv) << 4));
    }
    std::memcpy(b + 2, &sh, 2);
}

void encode_q4k(const float * x, uint8_t * b) {
    float sc[8], mn[8], smax = 0.f, mmax = 0.f;
    for (int i = 0; i < 8; ++i) {
        float lo = 0.f, hi = 0.f;  // the code range always holds zero
        for (int l = 0; l < 32; ++l) { lo = std::min(lo, x[32 * i + l]); hi = std::max(hi, x[32 * i + l]); }
        sc[i] = (hi - lo) / 15.f;
        mn[i] = -lo;
        smax = std::max(smax, sc[i]);
        mmax = std::max(mmax, mn[i]);
    }
    const uint16_t hd = tqo_float_to_half(smax / 63.f), hm = tqo_float_to_half(mmax / 63.f);
    const float d = tqo_half_to_float(hd), dm = tqo_half_to_float(hm);
    std::memset(b, 0, 144);
    std::memcpy(b, &hd, 2);
    std::memcpy(b + 2, &hm, 2);
    int s6[8], m6[8];
    for (int i = 0; i < 8; ++i) {
        s6[i] = d > 0.f ? std::min(63, std::max(0, int(std::nearbyint(sc[i] / d)))) : 0;
        m6[i] = dm > 0.f ? std::min(63, std::max(0, int(std::nearbyint(mn[i] / dm)))) : 0;
    }
    uint8_t * q = b + 4;
    for (int j = 0; j < 4; ++j) {
        q[j] = uint8_t(s6[j] | ((s6[j + 4] >> 4) << 6));
        q[j + 4] = uint8_t(m6[j] | ((m6[j + 4] >> 4) << 6));
        q[j + 8] = uint8_t((s6[j + 4] & 15) | ((m6[j + 4] & 15) << 4));
    }
    for (int c = 0; c < 4; ++c)
        for (int l = 0; l < 32; ++l) {
            int code[2];
            for (int h = 0; h < 2; ++h) {
                const int i = 2 * c + h;
                const float step = d * float(s6[i]), off = dm * float(m6[i]);
                const float v = x[64 * c + 32 * h + l];
                code[h] = step > 0.f ? std::min(15, std::max(0, int(std::nearbyint((v + off) / step)))) : 0;
            }
            b[16 + 32 * c + l] = uint8_t(code[0] | (code[1] << 4));
        }
}

void encode_q5k(const float * x, uint8_t * b) {  // encode_q4k with 32 levels and the high-bit plane
    float sc[8], mn[8], smax = 0.f, mmax = 0.f;
    for (int i = 0; i < 8; ++i) {
        float lo = 0.f, hi = 0.f;
        for (int l = 0; l < 32; ++l) { lo = std::min(lo, x[32 * i + l]); hi = std::max(hi, x[32 * i + l]); }
        sc[i] = (hi - lo) / 31.f;
        mn[i] = -lo;
        smax = std::max(smax, sc[i]);
        mmax = std::max(mmax, mn[i]);
    }
    const uint16_t hd = tqo_float_to_half(smax / 63.f), hm = tqo_float_to_half(mmax / 63.f);
    const float d = tqo_half_to_float(hd), dm = tqo_half_to_float(hm);
    std::memset(b, 0, 176);
    std::memcpy(b, &hd, 2);
    std::memcpy(b + 2, &hm, 2);
    int s6[8], m6[8];
    for (int i = 0; i < 8; ++i) {
        s6[i] = d > 0.f ? std::min(63, std::max(0, int(std::nearbyint(sc[i] / d)))) : 0;
        m6[i] = dm > 0.f ? std::min(63, std::max(0, int(std::nearbyint(mn[i] / dm)))) : 0;
    }
    uint8_t * q = b + 4;
    for (int j = 0; j < 4; ++j) {
        q[j] = uint8_t(s6[j] | ((s6[j + 4] >> 4) << 6));
        q[j + 4] = uint8_t(m6[j] | ((m6[j + 4] >> 4) << 6));
        q[j + 8] = uint8_t((s6[j + 4] & 15) | ((m6[j + 4] & 15) << 4));
    }
    for (int i = 0; i < 8; ++i)
        for (int l = 0; l < 32; ++l) {
            const float step = d * float(s6[i]), off = dm * float(m6[i]);
            const int code = step > 0.f ? std::min(31, std::max(0, int(std::nearbyint((x[32 * i + l] + off) / step)))) : 0;
            b[48 + 32 * (i / 2) + l] |= uint8_t((code & 15) << (4 * (i & 1)));
            b[16 + l] |= uint8_t((code >> 4) << i);
        }
}

void encode_q6k(const float * x, uint8_t * b) {  // 16 groups of 16: scale amax / 31, super scale max / 127
    float gs[16], big = 0.f;
    for (int g = 0; g < 16; ++g) {
        float amax = 0.f;
        for (int l = 0; l < 16; ++l) amax = std::max(amax, std::fabs(x[16 * g + l]));
        gs[g] = amax / 31.f;
        big = std::max(big, gs[g]);
    }
    const uint16_t hd = tqo_float_to_half(big / 127.f);
    const float d = tqo_half_to_float(hd);
    std::memset(b, 0, 210);
    std::memcpy(b + 208, &hd, 2);
    int code[256];
    for (int g = 0; g < 16; ++g) {
        const int sc = d > 0.f ? std::min(127, std::max(0, int(std::nearbyint(gs[g] / d)))) : 0;
        // weights 16 g .. of the block: sub-block i = g / 2 = 4 n + j, half is = g % 2: scale index 8 n + 2 j + is = g
        b[192 + g] = uint8_t(int8_t(sc));
        const float step = d * float(sc);
        for (int l = 0; l < 16; ++l)
            code[16 * g + l] = step > 0.f ? std::min(63, std::max(0, int(std::nearbyint(x[16 * g + l] / step)) + 32)) : 32;
    }
    for (int n = 0; n < 2; ++n)
        for (int l = 0; l < 32; ++l) {
            const int c0 = code[128 * n + l], c1 = code[128 * n + 32 + l], c2 = code[128 * n + 64 + l], c3 = code[128 * n + 96 + l];
            b[64 * n + l] = uint8_t((c0 & 15) | ((c2 & 15) << 4));
            b[64 * n + 32 + l] = uint8_t((c1 & 15) | ((c3 & 15) << 4));
            b[128 + 32 * n + l] = uint8_t((c0 >> 4) | ((c1 >> 4) << 2) | ((c2 >> 4) << 4) | ((c3 >> 4) << 6));
        }
}

// for every point of {0..7}^4 (12-bit code of magnitude levels) the nearest codebook point, lower index on a tie
const uint16_t * iq3s_nearest_table() {
    static std::vector<uint16_t> t;
    static std::once_flag once;
    std::call_once(once, [] {
        t.resize(4096);
        for (int c = 0; c < 4096; ++c) {
            int best = 0, bd = 1 << 30;
            for (int i = 0; i < 512; ++i) {
                const int g = tq_iq3s_lattice12[i];
                int dd = 0;
                for (int j = 0; j < 4; ++j) { const int df = ((c >> (3 * j)) & 7) - ((g >> (3 * j)) & 7); dd += df * df; }
                if (dd < bd) { bd = dd; best = i; }
            }
            t[size_t(c)] = uint16_t(best);
        }
    });
    return t.data();
}

// quantise 32 values with step db onto the codebook; returns the squared error, fills 8 point indices and 8 nibbles
float iq3s_fit(const float * x, float db, int * idx, int * sg) {
    const uint16_t * near = iq3s_nearest_table();
    const float inv = db > 0.f ? 1.f / db : 0.f;
    float err = 0.f;
    for (int w = 0; w < 8; ++w) {
        int code = 0, s = 0;
        for (int j = 0; j < 4; ++j) {
            const float v = x[4 * w + j];
            if (v < 0.f) s |= 1 << j;
            const int lev = std::min(7, std::max(0, int(std::nearbyint((std::fabs(v) * inv - 1.f) * 0.5f))));
            code |= lev << (3 * j);
        }
        idx[w] = near[code];
        sg[w] = s;
        const int g = tq_iq3s_lattice12[idx[w]];
        for (int j = 0; j < 4; ++j) {
            const float mag = db * float(2 * ((g >> (3 * j)) & 7) + 1);
            const float e = std::fabs(x[4 * w + j]) - mag;
            err += e * e;
        }
    }
    return err;
}

void encode_iq3s(const float * x, uint8_t * b) {
    float db[8], dmax = 0.f;
    int idx[8], sg[8];
    for (int ib = 0; ib < 8; ++ib) {
        float amax = 0.f;
        for (int i = 0; i < 32; ++i) amax = std::max(amax, std::fabs(x[32 * ib + i]));
        float best = 0.f, be = std::numeric_limits<float>::infinity();
        for (int c = 7; c <= 17; c += 2) {  // where on the magnitude ladder the largest value should sit
            const float cand = amax / float(c);
            const float e = iq3s_fit(x + 32 * ib, cand, idx, sg);
            if (e < be) { be = e; best = cand; }
        }
        db[ib] = best;
        dmax = std::max(dmax, best);
    }
    const uint16_t hd = tqo_float_to_half(dmax / 31.f);
    const float d = tqo_half_to_float(hd);
    std::memset(b, 0, 110);
    std::memcpy(b, &hd, 2);
    for (int ib = 0; ib < 8; ++ib) {
        int s = d > 0.f ? int(std::nearbyint((db[ib] / d - 1.f) * 0.5f)) : 0;
        s = std::min(15, std::max(0, s));
        b[106 + ib / 2] |= uint8_t(s << (4 * (ib & 1)));
        iq3s_fit(x + 32 * ib, d * float(1 + 2 * s), idx, sg);
        for (int w = 0; w < 8; ++w) {
            b[2 + 8 * ib + w] = uint8_t(idx[w] & 255);
            b[66 + ib] |= uint8_t((idx[w] >> 8) << w);
            b[74 + 4 * ib + w / 2] |= uint8_t(sg[w] << (4 * (w & 1)));
        }
    }
}

inline int nearest_e2m1(float v) {
    int best = 0;
    float bd = std::fabs(v);
    for (int i = 1; i < 16; ++i) {
        if (i == 8) continue;  // -0 is never emitted
        const float dd = std::fabs(v - kE2M1[i]);
        if (dd < bd) { bd = dd; best = i; }
    }
    return best;
}

void encode_nvfp4g_row(const float * x, uint8_t * b, int64_t cols) {
    float amax = 0.f;
    for (int64_t i = 0; i < cols; ++i) amax = std::max(amax, std::fabs(x[i]));
    const float g = amax > 0.f ? amax / (6.f * 448.f) : 1.f;  // the largest group scale lands on 448
    for (int64_t blk = 0; blk < cols / 128; ++blk, b += 76, x += 128) {
        std::memcpy(b, &g, 4);
        for (int grp = 0; grp < 8; ++grp) {
            float ga = 0.f;
            for (int i = 0; i < 16; ++i) ga = std::max(ga, std::fabs(x[16 * grp + i]));
            uint8_t sc = tqo_float_to_e4m3(ga / 6.f / g);
            if (ga > 0.f && sc == 0) sc = 1;
            b[4 + grp] = sc;
            const float d = tqo_e4m3_to_float(sc) * g, inv = d > 0.f ? 1.f / d : 0.f;
            for (int i = 0; i < 8; ++i)
                b[12 + 8 * grp + i] = uint8_t(nearest_e2m1(x[16 * grp + 2 * i] * inv) | (nearest_e2m1(x[16 * grp + 2 * i + 1] * inv) << 4));
        }
    }
}

}  // namespace

int tqo_quantize(uint32_t type, const float * src, void * dst, int64_t n, int64_t row) {
    int elems, bytes;
    if (!tqo_block_layout(type, &elems, &bytes) || n < 0 || n % elems) return -1;
    uint8_t * o = static_cast<uint8_t *>(dst);
    if (type == TQO_NVFP4G) {
        if (row <= 0 || row % 128 || n % row) return -1;
        for (int64_t r = 0; r < n / row; ++r) encode_nvfp4g_row(src + r * row, o + r * (row / 128) * 76, row);
        return 0;
    }
    for (int64_t b = 0; b < n / elems; ++b, src += elems, o += bytes) switch (type) {
        case TQO_Q4_K: encode_q4k(src, o); break;
        case TQO_Q5_K: encode_q5k(src, o); break;
        case TQO_Q6_K: encode_q6k(src, o); break;
        case TQO_IQ4_XS: encode_iq4xs(src, o); break;
        case TQO_IQ4_NL: encode_iq4nl(src, o); break;
        case TQO_Q8_0: encode_q8_0(src, o); break;
        case TQO_IQ3_S: encode_iq3s(src, o); break;
    }
    return 0;
}

// -------------------------------------------------------------------------------------------------- routing
namespace {
void gate_probs(int gating, int n, const float * logits, std::vector<float> & probs) {
    probs.resize(size_t(n));
    if (gating == TQO_GATE_SOFTMAX) {  // src/experts/moe.cpp:35-44: max, exp(l - max) summed in index order, divide
        float mx = -INFINITY;
        for (int i = 0; i < n; ++i) mx = std::max(mx, logits[i]);
        float sum = 0.f;
        for (int i = 0; i < n; ++i) { probs[size_t(i)] = std::exp(logits[i] - mx); sum += probs[size_t(i)]; }
        for (int i = 0; i < n; ++i) probs[size_t(i)] /= sum;
    } else if (gating == TQO_GATE_SIGMOID) {  // src/experts/moe.cpp:10-14
        for (int i = 0; i < n; ++i) probs[size_t(i)] = 1.0f / (1.0f + std::exp(-logits[i]));
    } else if (gating == TQO_GATE_SOFTMAX_WEIGHT) {  // src/experts/moe.cpp:48-50: the raw logits; softmax comes after the choice
        for (int i = 0; i < n; ++i) probs[size_t(i)] = logits[i];
    } else {  // sqrt(softplus), src/experts/moe.cpp:15-19 and 51-53
        for (int i = 0; i < n; ++i) {
            const float x = logits[i];
            const float sp = x > 0.f ? x + std::log1p(std::exp(-x)) : std::log1p(std::exp(x));
            probs[size_t(i)] = std::sqrt(sp);
        }
    }
}
}  // namespace

int tqo_route(int gating, int n_expert, int k, int norm_weights, float weight_scale, const float * logits,
              const float * bias, int32_t * ids, float * weights) {
    if (n_expert <= 0 || k <= 0 || k > n_expert) return -1;
    if (gating < TQO_GATE_SOFTMAX || gating > TQO_GATE_SQRT_SOFTPLUS) return -1;
    std::vector<float> probs;
    gate_probs(gating, n_expert, logits, probs);
    std::vector<float> sel(probs);  // selection values: bias added for the choice only (moe.cpp:63-65)
    if (bias) for (int i = 0; i < n_expert; ++i) sel[size_t(i)] += bias[i];
    std::vector<int> order(static_cast<size_t>(n_expert));
    std::iota(order.begin(), order.end(), 0);
    std::stable_sort(order.begin(), order.end(), [&](int a, int b) {  // moe.cpp:73-78
        if (sel[size_t(a)] != sel[size_t(b)]) return sel[size_t(a)] > sel[size_t(b)];
        return a < b;
    });
    for (int s = 0; s < k; ++s) { ids[s] = order[size_t(s)]; weights[s] = probs[size_t(order[size_t(s)])]; }
    if (gating == TQO_GATE_SOFTMAX_WEIGHT) {  // moe.cpp:88-97: softmax over the selected weights only
        float mx = -INFINITY;
        for (int s = 0; s < k; ++s) mx = std::max(mx, weights[s]);
        float sum = 0.f;
        for (int s = 0; s < k; ++s) { weights[s] = std::exp(weights[s] - mx); sum += weights[s]; }
        for (int s = 0; s < k; ++s) weights[s] /= sum;
    }
    if (norm_weights) {  // moe.cpp:101-106
        float sum = 0.f;
        for (int s = 0; s < k; ++s) sum += weights[s];
        sum = std::max(sum, 6.103515625e-5f);
        for (int s = 0; s < k; ++s) weights[s] /= sum;
    }
    if (weight_scale != 0.f && weight_scale != 1.f) for (int s = 0; s < k; ++s) weights[s] *= weight_scale;
    return 0;
}

int tqo_route_softmax_collision(int n_expert, int k, const float * logits) {
    std::vector<float> probs;
    gate_probs(TQO_GATE_SOFTMAX, n_expert, logits, probs);
    std::vector<int> order(static_cast<size_t>(n_expert));
    std::iota(order.begin(), order.end(), 0);
    std::stable_sort(order.begin(), order.end(), [&](int a, int b) {
        if (probs[size_t(a)] != probs[size_t(b)]) return probs[size_t(a)] > probs[size_t(b)];
        return a < b;
    });
    int found = 0;
    for (int s = 0; s < k && s + 1 < n_expert; ++s) {
        const int a = order[size_t(s)], b = order[size_t(s) + 1];
        const float pa = probs[size_t(a)], pb = probs[size_t(b)];
        // a probability below the smallest normal number sits where exp() implementations flush differently
        if ((pa != 0.f && pa < 1.17549435e-38f) || (pb != 0.f && pb < 1.17549435e-38f)) found = 1;
        if (pa == pb && pa != 0.f && logits[a] != logits[b]) found = 1;
    }
    return found;
}

float tqo_shared_weight(float logit) { return 1.f / (1.f + std::exp(-logit)); }

int tqo_dispatch(const int32_t * ids, int A, int E, int32_t * counts, int32_t * offsets, int32_t * perm) {
    if (A < 0 || E <= 0) return -1;
    for (int e = 0; e < E; ++e) counts[e] = 0;
    for (int a = 0; a < A; ++a) {
        if (ids[a] >= E) return -1;
        if (ids[a] >= 0) ++counts[ids[a]];
    }
    offsets[0] = 0;
    for (int e = 0; e < E; ++e) offsets[e + 1] = offsets[e] + counts[e];
    std::vector<int32_t> fill(offsets, offsets + E);
    for (int a = 0; a < A; ++a) if (ids[a] >= 0) perm[fill[size_t(ids[a])]++] = a;  // ascending a inside an expert
    return 0;
}

// ------------------------------------------------------------------------- residual add and RMS norm before the layer
namespace {
// __shfl_xor butterfly over 32 lanes with offsets 16, 8, 4, 2, 1: every lane ends with the same value
float butterfly32(float * v) {
    for (int o = 16; o; o >>= 1) {
        float t[32];
        for (int i = 0; i < 32; ++i) t[i] = v[i] + v[i ^ o];
        for (int i = 0; i < 32; ++i) v[i] = t[i];
    }
    return v[0];
}
}  // namespace

int tqo_add_rmsnorm(uint16_t * rows, const uint16_t * residual, const float * weight, float eps, int hidden, int n,
                    uint16_t * normed_bf16) {
    if (hidden <= 0 || hidden % 256 || n <= 0) return -1;
    const int nparts = hidden / 256;
    std::vector<float> partial(static_cast<size_t>(nparts));
    for (int t = 0; t < n; ++t) {
        uint16_t * m = rows + size_t(t) * hidden;
        for (int b = 0; b < nparts; ++b) {  // quant_tq3.inc:303-313 with block_sum256 (:293-301)
            float warp_sum[8];
            for (int w = 0; w < 8; ++w) {
                float sq[32];
                for (int l = 0; l < 32; ++l) {
                    const int i = b * 256 + w * 32 + l;
                    if (residual) m[i] = tqo_float_to_bf16(tqo_bf16_to_float(m[i]) + tqo_bf16_to_float(residual[size_t(t) * hidden + i]));
                    const float v = tqo_bf16_to_float(m[i]);
                    sq[l] = v * v;
                }
                warp_sum[w] = butterfly32(sq);
            }
            float s = 0.f;
            for (int w = 0; w < 8; ++w) s += warp_sum[w];
            partial[size_t(b)] = s;
        }
        float lanes[32];  // quant.cu:651-656
        for (int l = 0; l < 32; ++l) {
            float s = 0.f;
            for (int i = l; i < nparts; i += 32) s += partial[size_t(i)];
            lanes[l] = s;
        }
        const float total = butterfly32(lanes);
        const float inv = 1.0f / std::sqrt(total / float(hidden) + eps);
        for (int i = 0; i < hidden; ++i)  // quant.cu:660: rounded to bf16 whatever the storage
            normed_bf16[size_t(t) * hidden + i] = tqo_float_to_bf16(tqo_bf16_to_float(m[i]) * inv * weight[i]);
    }
    return 0;
}

// -------------------------------------------------------------------------------------------- FFN and combine
void tqo_expert_ffn(const float * x, int hidden, const float * w_gate, const float * w_up, const float * w_down,
                    int ff, float swiglu_clamp, int clamp_gate, float * out) {
    std::vector<float> act(size_t(ff), 0.f);
    for (int o = 0; o < ff; ++o) {  // moe.cpp:119-128: fp32 sums in column order
        float g = 0.f, u = 0.f;
        const float * wg = w_gate + size_t(o) * hidden, * wu = w_up + size_t(o) * hidden;
        for (int i = 0; i < hidden; ++i) { g += wg[i] * x[i]; u += wu[i] * x[i]; }
        if (swiglu_clamp > 1e-6f) {  // moe.cpp:133-143
            u = std::min(std::max(u, -swiglu_clamp), swiglu_clamp);
            if (clamp_gate) g = std::min(g, swiglu_clamp);
            float s = g / (1.f + std::exp(-g));
            if (!clamp_gate) s = std::min(s, swiglu_clamp);
            act[size_t(o)] = s * u;
        } else {
            act[size_t(o)] = (g / (1.f + std::exp(-g))) * u;
        }
    }
    for (int i = 0; i < hidden; ++i) {
        float s = 0.f;
        const float * wd = w_down + size_t(i) * ff;
        for (int o = 0; o < ff; ++o) s += wd[o] * act[size_t(o)];
        out[i] = s;
    }
}

void tqo_combine(const int k, const float * weights, const float * expert_outs, int hidden, float * out) {
    for (int s = 0; s < k; ++s)
        for (int i = 0; i < hidden; ++i) out[i] += weights[s] * expert_outs[size_t(s) * hidden + i];
}

namespace {
inline float load_as_float(const void * p, uint32_t type, size_t i) {
    switch (type) {
        case TQO_F32: return static_cast<const float *>(p)[i];
        case TQO_BF16: return tqo_bf16_to_float(static_cast<const uint16_t *>(p)[i]);
        default: return tqo_half_to_float(static_cast<const uint16_t *>(p)[i]);
    }
}
}  // namespace

int tqo_router_logits(const void * w, uint32_t wtype, const void * shared_gate, const void * x, uint32_t xtype,
                      int hidden, int E, int n, float * logits) {
    if (hidden <= 0 || E <= 0 || n <= 0) return -1;
    for (uint32_t t : {wtype, xtype}) if (t != TQO_F32 && t != TQO_BF16 && t != TQO_F16) return -1;
    for (int t = 0; t < n; ++t)
        for (int r = 0; r <= E; ++r) {
            float sum = 0.f;
            if (r < E || shared_gate) {
                const void * row = r < E ? w : shared_gate;
                const size_t base = r < E ? size_t(r) * hidden : 0;
                for (int j = 0; j < hidden; ++j)
                    sum += load_as_float(row, wtype, base + j) * load_as_float(x, xtype, size_t(t) * hidden + j);
            }
            logits[size_t(t) * (E + 1) + r] = sum;
        }
    return 0;
}

// --------------------------------------------------------------------------------- declared operand quantisers
void tqo_quant_act_row_i8(const float * x, int cols, int8_t * q, float * scale) {
    float m = 0.f;
    for (int i = 0; i < cols; ++i) m = std::max(m, std::fabs(x[i]));
    *scale = m / 127.f;
    const float mul = m > 0.f ? 127.f / m : 0.f;
    for (int i = 0; i < cols; ++i) q[i] = int8_t(std::nearbyint(x[i] * mul));
}

// reference: quant_act_rows_k<false> (src/formats/weight/quant_u4h.inc:790-822): a scale per 32 values (amax / 127 of the
// block), q = rint(x * (127 / amax)), and the sum of q over each half of 16 (the weights' "min" term of the int8 products)
void tqo_quant_act_blocks_i8(const float * x, int cols, int8_t * q, float * scales, int16_t * qsum) {
    for (int b = 0; b < cols / 32; ++b) {
        tqo_quant_act_row_i8(x + 32 * b, 32, q + 32 * b, scales + b);
        if (qsum)
            for (int h = 0; h < 2; ++h) {
                int sum = 0;
                for (int i = 0; i < 16; ++i) sum += q[32 * b + 16 * h + i];
                qsum[2 * b + h] = int16_t(sum);
            }
    }
}

void tqo_quant_act_row_e4m3(const float * x, int cols, uint8_t * q, float * scale) {
    float m = 0.f;
    for (int i = 0; i < cols; ++i) m = std::max(m, std::fabs(x[i]));
    *scale = m / 448.f;
    const float mul = m > 0.f ? 448.f / m : 0.f;
    for (int i = 0; i < cols; ++i) q[i] = tqo_float_to_e4m3(x[i] * mul);
}

// ------------------------------------------------------------------------------------------------ whole layer
namespace {

void requant_row_i8(float * x, int cols) {  // x <- dequantised per-row int8 image of x
    std::vector<int8_t> q(static_cast<size_t>(cols));
    float s;
    tqo_quant_act_row_i8(x, cols, q.data(), &s);
    for (int i = 0; i < cols; ++i) x[i] = float(q[size_t(i)]) * s;
}

void requant_row_e4m3(float * x, int cols) {  // x <- dequantised per-row E4M3 image of x
    std::vector<uint8_t> q(static_cast<size_t>(cols));
    float s;
    tqo_quant_act_row_e4m3(x, cols, q.data(), &s);
    for (int i = 0; i < cols; ++i) x[i] = tqo_e4m3_to_float(q[size_t(i)]) * s;
}
void requant_row(int act_mode, float * x, int cols) {
    if (act_mode == 2) requant_row_e4m3(x, cols);
    else if (act_mode == 6) for (int b = 0; b < cols / 32; ++b) requant_row_i8(x + 32 * b, 32);   // a scale per 32 values
    else requant_row_i8(x, cols);
}
// act_mode 2 reads the banks as the fp8 products do
int decode_weights(const tqo_layer & L, uint32_t type, const void * src, float * dst, int64_t n) {
    return L.act_mode == 2 ? tqo_dequantize_nvfp4_widened(src, dst, n) : tqo_dequantize(type, src, dst, n);
}

struct Decoded { std::vector<float> gate, up, down; };

int decode_expert(const tqo_layer & L, int e, int ff, Decoded & d) {
    int elems, bytes;
    tqo_block_layout(L.wtype, &elems, &bytes);
    const int64_t gu = int64_t(L.ff) * L.hidden;           // weights of one stacked expert matrix
    const size_t stride = size_t(gu / elems) * bytes;      // bytes of one expert in a bank
    d.gate.resize(size_t(ff) * L.hidden);
    d.up.resize(size_t(ff) * L.hidden);
    d.down.resize(size_t(L.hidden) * ff);
    // gate / up: the first ff rows of expert e
    if (decode_weights(L, L.wtype, static_cast<const uint8_t *>(L.gate) + stride * e, d.gate.data(), int64_t(ff) * L.hidden)) return -1;
    if (decode_weights(L, L.wtype, static_cast<const uint8_t *>(L.up) + stride * e, d.up.data(), int64_t(ff) * L.hidden)) return -1;
    // down: rows of L.ff columns, the first ff columns kept; its bank may have a format of its own
    const uint32_t dtype = L.wtype_down ? L.wtype_down : L.wtype;
    int delems, dbytes;
    if (!tqo_block_layout(dtype, &delems, &dbytes) || L.ff % delems) return -1;
    std::vector<float> row(static_cast<size_t>(L.ff));
    const size_t row_bytes = size_t(L.ff / delems) * dbytes, dstride = size_t(gu / delems) * dbytes;
    for (int r = 0; r < L.hidden; ++r) {
        if (decode_weights(L, dtype, static_cast<const uint8_t *>(L.down) + dstride * e + row_bytes * r, row.data(), L.ff)) return -1;
        std::copy(row.begin(), row.begin() + ff, d.down.begin() + size_t(r) * ff);
    }
    return 0;
}

// FFN with the declared activation quantiser applied to both matvec inputs
void ffn_mode(const tqo_layer & L, const float * x, const Decoded & d, int ff, float * out, float * act_out = nullptr) {
    if (L.act_mode == 0) { tqo_expert_ffn(x, L.hidden, d.gate.data(), d.up.data(), d.down.data(), ff, L.swiglu_clamp, L.clamp_gate, out); return; }
    std::vector<float> act(static_cast<size_t>(ff));
    const float limit = L.swiglu_clamp;
    const bool clamp = limit > 1e-6f;   // src/experts/moe.cpp:128-143, as tqo_expert_ffn
    for (int o = 0; o < ff; ++o) {
        float g = 0.f, u = 0.f;
        const float * wg = d.gate.data() + size_t(o) * L.hidden, * wu = d.up.data() + size_t(o) * L.hidden;
        for (int i = 0; i < L.hidden; ++i) { g += wg[i] * x[i]; u += wu[i] * x[i]; }
        if (clamp) {
            u = std::min(std::max(u, -limit), limit);
            if (L.clamp_gate) g = std::min(g, limit);
        }
        float s = g / (1.f + std::exp(-g));
        if (clamp && !L.clamp_gate) s = std::min(s, limit);
        act[size_t(o)] = s * u;
    }
    const bool f16 = L.act_mode == 5 || L.act_mode == 2 || L.act_mode == 6;   // the grouped products keep act and y as fp16 rows
    if (f16) for (float & v : act) v = tqo_half_to_float(tqo_float_to_half(v));
    if (act_out) std::copy(act.begin(), act.end(), act_out);
    requant_row(L.act_mode, act.data(), ff);
    for (int i = 0; i < L.hidden; ++i) {
        float s = 0.f;
        const float * wd = d.down.data() + size_t(i) * ff;
        for (int o = 0; o < ff; ++o) s += wd[o] * act[size_t(o)];
        out[i] = f16 ? tqo_half_to_float(tqo_float_to_half(s)) : s;
    }
}

}  // namespace

int tqo_layer_forward(const tqo_layer * Lp, const float * x, const float * logits, int n, float * out,
                      int32_t * ids_out, float * weights_out) {
    const tqo_layer & L = *Lp;
    int elems, bytes;
    if (!tqo_block_layout(L.wtype, &elems, &bytes)) return -1;
    if (L.hidden % elems || L.ff % elems || n <= 0 || L.k <= 0 || L.k > L.n_expert) return -1;
    if (L.act_mode != 0 && L.act_mode != 1 && L.act_mode != 2 && L.act_mode != 5 && L.act_mode != 6) return -1;
    if (L.act_mode == 6 && (L.hidden % 32 || L.ff % 32 || (L.has_shared && L.shared_ff % 32))) return -1;
    if (L.act_mode == 2 && (L.wtype != TQO_NVFP4G || (L.wtype_down && L.wtype_down != TQO_NVFP4G))) return -1;
    if (L.has_shared && (L.shared_ff <= 0 || L.shared_ff > L.ff || L.shared_ff % elems)) return -1;
    const int E = L.n_expert, K = L.k, A = n * K, H = L.hidden;
    std::vector<int32_t> ids(static_cast<size_t>(A)), counts(static_cast<size_t>(E)), offsets(size_t(E) + 1), perm(static_cast<size_t>(A));
    std::vector<float> weights(static_cast<size_t>(A));
    for (int t = 0; t < n; ++t)
        if (tqo_route(L.gating ? L.gating : int(TQO_GATE_SOFTMAX), E, K, L.raw_weights ? 0 : 1, L.weight_scale, logits + size_t(t) * (E + 1), L.bias,
                      ids.data() + size_t(t) * K, weights.data() + size_t(t) * K)) return -1;
    tqo_dispatch(ids.data(), A, E, counts.data(), offsets.data(), perm.data());
    if (ids_out) std::copy(ids.begin(), ids.end(), ids_out);
    if (weights_out) std::copy(weights.begin(), weights.end(), weights_out);

    std::vector<float> xin(x, x + size_t(n) * H);
    if (L.act_mode) for (int t = 0; t < n; ++t) requant_row(L.act_mode, xin.data() + size_t(t) * H, H);

    std::vector<float> routed(size_t(A) * H), shared(L.has_shared ? size_t(n) * H : 0);
    std::atomic<int> next{0}, failed{0};
    const int jobs = E + (L.has_shared ? 1 : 0);
    auto worker = [&]() {
        Decoded d;
        for (;;) {
            const int e = next.fetch_add(1);
            if (e >= jobs) break;
            if (e < E) {
                if (!counts[size_t(e)]) continue;
                if (decode_expert(L, e, L.ff, d)) { failed = 1; continue; }
                for (int i = offsets[size_t(e)]; i < offsets[size_t(e) + 1]; ++i) {
                    const int a = perm[size_t(i)];
                    const size_t arow = size_t(a / K) * size_t(K + (L.has_shared ? 1 : 0)) + size_t(a % K);
                    ffn_mode(L, xin.data() + size_t(a / K) * H, d, L.ff, routed.data() + size_t(a) * H, L.act_out ? L.act_out + arow * L.ff : nullptr);
                }
            } else {
                if (decode_expert(L, E, L.shared_ff, d)) { failed = 1; continue; }
                for (int t = 0; t < n; ++t)
                    ffn_mode(L, xin.data() + size_t(t) * H, d, L.shared_ff, shared.data() + size_t(t) * H,
                             L.act_out ? L.act_out + (size_t(t) * size_t(K + 1) + size_t(K)) * L.ff : nullptr);
            }
        }
    };
    const int nt = std::max(1, L.threads);
    std::vector<std::thread> pool;
    for (int i = 1; i < nt; ++i) pool.emplace_back(worker);
    worker();
    for (auto & th : pool) th.join();
    if (failed) return -1;

    for (int t = 0; t < n; ++t) {  // src/experts/moe.cu:224-234: slots in order, then the shared row
        float * o = out + size_t(t) * H;
        std::fill(o, o + H, 0.f);
        tqo_combine(K, weights.data() + size_t(t) * K, routed.data() + size_t(t) * K * H, H, o);
        if (L.has_shared) {
            const float sw = tqo_shared_weight(logits[size_t(t) * (E + 1) + E]);
            for (int i = 0; i < H; ++i) o[i] += sw * shared[size_t(t) * H + i];
        }
    }
    return 0;
}

// ---------------------------------------------------------------------------------------------- CPU baseline
// Scheme of the reference's tests/bench_cpu_expert_mt.cpp: table 1 (:69-116) has workers pull whole experts from an
// atomic counter, gate -> up -> down per expert, one warm pass, `reps` timed passes, for thread counts 1, 2, 4, ...;
// table 2 (:130-199) splits the rows of ONE expert's three matrices over persistent workers woken by a generation
// counter (single-expert latency). Both on this build's bank formats. The int8 variant quantises the input per
// 32-block (scale amax / 127) and takes integer dots with the block's integer codes on AVX2 (unsigned x signed byte
// products summed in pairs, then widened: the instruction pair the reference's K-quant dots use,
// src/experts/cpu_kquant.cpp:85-101, 154-172; its IQ4_NL kernel, src/experts/cpu_expert_matvec.cpp:200-280, takes the
// 16-bit route to the same sums). The fp32 variant decodes a block and multiplies in fp32 (eight partial sums).
namespace {

// integer image of one 32-weight block: w[i] = scale[i / 16] * q[i] + offset
struct BlockI8 { int8_t q[32]; float scale[2], offset; };

// scalar decode of a block's integer codes: every format the baseline runs (the vector decoders below are checked against it)
inline void block_image(uint32_t type, const uint8_t * blk, int ib, BlockI8 & o) {
    o.offset = 0.f;
    switch (type) {
        case TQO_IQ4_XS: {
            o.scale[0] = o.scale[1] = tqo_half_to_float(rd16(blk)) * float(iq4xs_subscale(blk, ib) - 32);
            const uint8_t * q = blk + 8 + 16 * ib;
            for (int j = 0; j < 16; ++j) { o.q[j] = kIq4Values[q[j] & 15]; o.q[16 + j] = kIq4Values[q[j] >> 4]; }
            break;
        }
        case TQO_IQ4_NL: {
            o.scale[0] = o.scale[1] = tqo_half_to_float(rd16(blk));
            for (int j = 0; j < 16; ++j) { o.q[j] = kIq4Values[blk[2 + j] & 15]; o.q[16 + j] = kIq4Values[blk[2 + j] >> 4]; }
            break;
        }
        case TQO_Q4_K: {
            int sc, mn;
            q4k_scale_min(blk + 4, ib, sc, mn);
            o.scale[0] = o.scale[1] = tqo_half_to_float(rd16(blk)) * float(sc);
            o.offset = -(tqo_half_to_float(rd16(blk + 2)) * float(mn));
            const uint8_t * q = blk + 16 + 32 * (ib / 2);
            for (int l = 0; l < 32; ++l) o.q[l] = int8_t((ib & 1) ? q[l] >> 4 : q[l] & 15);
            break;
        }
        case TQO_IQ3_S: {
            o.scale[0] = o.scale[1] = tqo_half_to_float(rd16(blk)) * float(1 + 2 * ((blk[106 + ib / 2] >> (4 * (ib & 1))) & 15));
            for (int w = 0; w < 8; ++w) {
                const uint32_t g = tq_iq3s_point(blk[2 + 8 * ib + w] | (((blk[66 + ib] >> w) & 1) << 8));
                const int sg = blk[74 + 4 * ib + w / 2] >> (4 * (w & 1));
                for (int j = 0; j < 4; ++j) { const int m = (g >> (8 * j)) & 255; o.q[4 * w + j] = int8_t(((sg >> j) & 1) ? -m : m); }
            }
            break;
        }
        default: {  // NVFP4G (128-weight block): q = 2 * e2m1, one scale per 16 weights
            float g;
            std::memcpy(&g, blk, 4);
            for (int h = 0; h < 2; ++h) {
                o.scale[h] = 0.5f * (tqo_e4m3_to_float(blk[4 + 2 * ib + h]) * g);
                for (int i = 0; i < 8; ++i) {
                    const uint8_t c = blk[12 + 8 * (2 * ib + h) + i];
                    o.q[16 * h + 2 * i] = int8_t(std::lrintf(2.f * kE2M1[c & 15]));
                    o.q[16 * h + 2 * i + 1] = int8_t(std::lrintf(2.f * kE2M1[c >> 4]));
                }
            }
        }
    }
}

// the same block as a 32-byte vector (AVX2)
struct Iq3Table { uint32_t v[512]; Iq3Table() { for (int i = 0; i < 512; ++i) v[i] = tq_iq3s_point(i); } };
inline __m256i block_codes_avx2(uint32_t type, const uint8_t * blk, int ib) {
    switch (type) {
        case TQO_IQ4_XS: case TQO_IQ4_NL: {
            const __m128i table = _mm_loadu_si128(reinterpret_cast<const __m128i *>(kIq4Values));
            const __m128i q = _mm_loadu_si128(reinterpret_cast<const __m128i *>(type == TQO_IQ4_XS ? blk + 8 + 16 * ib : blk + 2));
            const __m128i m4 = _mm_set1_epi8(15);
            return _mm256_set_m128i(_mm_shuffle_epi8(table, _mm_and_si128(_mm_srli_epi16(q, 4), m4)), _mm_shuffle_epi8(table, _mm_and_si128(q, m4)));
        }
        case TQO_Q4_K: {
            const __m256i q = _mm256_loadu_si256(reinterpret_cast<const __m256i *>(blk + 16 + 32 * (ib / 2)));
            return _mm256_and_si256((ib & 1) ? _mm256_srli_epi16(q, 4) : q, _mm256_set1_epi8(15));
        }
        case TQO_IQ3_S: {
            static const Iq3Table table;
            // eight lattice indices: the byte, and bit w of the sub-block's qh byte as bit 8
            const __m256i low = _mm256_cvtepu8_epi32(_mm_loadl_epi64(reinterpret_cast<const __m128i *>(blk + 2 + 8 * ib)));
            const __m256i bit = _mm256_and_si256(_mm256_srlv_epi32(_mm256_set1_epi32(blk[66 + ib]), _mm256_setr_epi32(0, 1, 2, 3, 4, 5, 6, 7)), _mm256_set1_epi32(1));
            const __m256i mag = _mm256_i32gather_epi32(reinterpret_cast<const int *>(table.v), _mm256_or_si256(low, _mm256_slli_epi32(bit, 8)), 4);
            // sign bit 4 w + j of the sub-block's 32 sign bits belongs to byte 4 w + j: spread the four sign bytes over the
            // vector, pick each byte's bit, and negate where it is set
            uint32_t sg;
            std::memcpy(&sg, blk + 74 + 4 * ib, 4);
            const __m256i bytes = _mm256_shuffle_epi8(_mm256_set1_epi32(int(sg)), _mm256_setr_epi8(0, 0, 0, 0, 0, 0, 0, 0, 1, 1, 1, 1, 1, 1, 1, 1, 2, 2, 2, 2, 2, 2, 2, 2, 3, 3, 3, 3, 3, 3, 3, 3));
            const __m256i pick = _mm256_set1_epi64x(int64_t(0x8040201008040201ull));
            const __m256i neg = _mm256_cmpeq_epi8(_mm256_and_si256(bytes, pick), pick);
            return _mm256_sub_epi8(_mm256_xor_si256(mag, neg), neg);
        }
        default: {  // NVFP4G: byte i of a group = weights 2 i (low nibble) and 2 i + 1
            static const int8_t two_e2m1[16] = {0, 1, 2, 3, 4, 6, 8, 12, 0, -1, -2, -3, -4, -6, -8, -12};
            const __m128i table = _mm_loadu_si128(reinterpret_cast<const __m128i *>(two_e2m1));
            const __m128i q = _mm_loadu_si128(reinterpret_cast<const __m128i *>(blk + 12 + 16 * ib));
            const __m128i m4 = _mm_set1_epi8(15);
            const __m128i even = _mm_shuffle_epi8(table, _mm_and_si128(q, m4)), odd = _mm_shuffle_epi8(table, _mm_and_si128(_mm_srli_epi16(q, 4), m4));
            return _mm256_set_m128i(_mm_unpackhi_epi8(even, odd), _mm_unpacklo_epi8(even, odd));
        }
    }
}
inline float half_hw(const uint8_t * p) { return _cvtsh_ss(rd16(p)); }   // the hardware conversion (equal to tqo_half_to_float on all 65,536 halves)
inline void block_scales(uint32_t type, const uint8_t * blk, int ib, float (&scale)[2], float & offset) {
    offset = 0.f;
    switch (type) {
        case TQO_IQ4_XS: scale[0] = scale[1] = half_hw(blk) * float(iq4xs_subscale(blk, ib) - 32); break;
        case TQO_IQ4_NL: scale[0] = scale[1] = half_hw(blk); break;
        case TQO_Q4_K: {
            int sc, mn;
            q4k_scale_min(blk + 4, ib, sc, mn);
            scale[0] = scale[1] = half_hw(blk) * float(sc);
            offset = -(half_hw(blk + 2) * float(mn));
            break;
        }
        case TQO_IQ3_S: scale[0] = scale[1] = half_hw(blk) * float(1 + 2 * ((blk[106 + ib / 2] >> (4 * (ib & 1))) & 15)); break;
        default: {
            float g;
            std::memcpy(&g, blk, 4);
            for (int h = 0; h < 2; ++h) scale[h] = 0.5f * (tqo_e4m3_to_float(blk[4 + 2 * ib + h]) * g);
        }
    }
}

struct XQ { std::vector<int8_t> q; std::vector<float> scale; std::vector<int> sum; };

void quant_x_blocks(const float * x, int cols, XQ & o) {
    o.q.resize(static_cast<size_t>(cols));
    o.scale.resize(size_t(cols / 32));
    o.sum.resize(size_t(cols / 32));
    for (int b = 0; b < cols / 32; ++b) {
        float m = 0.f;
        for (int i = 0; i < 32; ++i) m = std::max(m, std::fabs(x[32 * b + i]));
        o.scale[size_t(b)] = m / 127.f;
        const float mul = m > 0.f ? 127.f / m : 0.f;
        int s = 0;
        for (int i = 0; i < 32; ++i) { const int v = int(std::nearbyint(x[32 * b + i] * mul)); o.q[size_t(32 * b + i)] = int8_t(v); s += v; }
        o.sum[size_t(b)] = s;
    }
}

inline float hsum8(__m256 v) {
    __m128 s = _mm_add_ps(_mm256_castps256_ps128(v), _mm256_extractf128_ps(v, 1));
    s = _mm_add_ps(s, _mm_movehl_ps(s, s));
    s = _mm_add_ss(s, _mm_shuffle_ps(s, s, 1));
    return _mm_cvtss_f32(s);
}

// rows [r0, r1) of y = W x. mode 0: fp32 (decode, fp32 products, eight partial sums); 1: int8 activations, AVX2 integer
// dots; 2: int8 activations, scalar integer dots (the check of mode 1)
__attribute__((optimize("O3"))) void matvec_rows(uint32_t type, const uint8_t * W, int cols, const float * x, const XQ * xq, int mode, int r0, int r1, float * y) {
    int elems, bytes;
    tqo_block_layout(type, &elems, &bytes);
    const size_t row_bytes = size_t(cols / elems) * bytes;
    const __m256i ones = _mm256_set1_epi16(1);
    std::vector<float> xsum;   // fp32 path: the sum of every 32-block of x (what a block's offset multiplies)
    if (mode == 0) {
        xsum.resize(size_t(cols / 32));
        for (int b = 0; b < cols / 32; ++b) { float t = 0.f; for (int i = 0; i < 32; ++i) t += x[32 * b + i]; xsum[size_t(b)] = t; }
    }
    for (int r = r0; r < r1; ++r) {
        const uint8_t * row = W + row_bytes * r;
        float result;
        if (mode == 1) {
            __m256 acc = _mm256_setzero_ps();
            float off = 0.f;
            for (int b = 0; b < cols / 32; ++b) {
                const uint8_t * blk = row + size_t((32 * b) / elems) * bytes;
                const int ib = (32 * b % elems) / 32;
                float sc[2], offset;
                block_scales(type, blk, ib, sc, offset);
                const __m256i w = block_codes_avx2(type, blk, ib);
                const __m256i q = _mm256_loadu_si256(reinterpret_cast<const __m256i *>(xq->q.data() + 32 * b));
                // |w| as the unsigned operand, q with w's sign as the signed one: pair sums stay below 2^15 (|w|, |q| <= 127)
                const __m256i dot = _mm256_madd_epi16(_mm256_maddubs_epi16(_mm256_sign_epi8(w, w), _mm256_sign_epi8(q, w)), ones);
                const float xs = xq->scale[size_t(b)];
                const __m256 scale = _mm256_set_m128(_mm_set1_ps(sc[1] * xs), _mm_set1_ps(sc[0] * xs));   // weights 0..15 in the low half
                acc = _mm256_fmadd_ps(_mm256_cvtepi32_ps(dot), scale, acc);
                off += offset * (xs * float(xq->sum[size_t(b)]));
            }
            result = hsum8(acc) + off;
        } else if (mode == 2) {
            float acc = 0.f;
            BlockI8 bi;
            for (int b = 0; b < cols / 32; ++b) {
                const uint8_t * blk = row + size_t((32 * b) / elems) * bytes;
                block_image(type, blk, (32 * b % elems) / 32, bi);
                const int8_t * q = xq->q.data() + 32 * b;
                int d0 = 0, d1 = 0;
                for (int i = 0; i < 16; ++i) { d0 += int(bi.q[i]) * int(q[i]); d1 += int(bi.q[16 + i]) * int(q[16 + i]); }
                acc += xq->scale[size_t(b)] * (bi.scale[0] * float(d0) + bi.scale[1] * float(d1) + bi.offset * float(xq->sum[size_t(b)]));
            }
            result = acc;
        } else {
            // fp32: the block's integer codes widened to fp32, four fused multiply-adds of eight products each, then the block's
            // scale (w = scale * q + offset, so the offset meets the plain sum of the block's x)
            __m256 acc = _mm256_setzero_ps();
            float off = 0.f;
            for (int b = 0; b < cols / 32; ++b) {
                const uint8_t * blk = row + size_t((32 * b) / elems) * bytes;
                const int ib = (32 * b % elems) / 32;
                float sc[2], offset;
                block_scales(type, blk, ib, sc, offset);
                const __m256i w = block_codes_avx2(type, blk, ib);
                const __m128i lo = _mm256_castsi256_si128(w), hi = _mm256_extracti128_si256(w, 1);
                const float * xb = x + 32 * b;
                __m256 p0 = _mm256_mul_ps(_mm256_cvtepi32_ps(_mm256_cvtepi8_epi32(lo)), _mm256_loadu_ps(xb));
                p0 = _mm256_fmadd_ps(_mm256_cvtepi32_ps(_mm256_cvtepi8_epi32(_mm_srli_si128(lo, 8))), _mm256_loadu_ps(xb + 8), p0);
                __m256 p1 = _mm256_mul_ps(_mm256_cvtepi32_ps(_mm256_cvtepi8_epi32(hi)), _mm256_loadu_ps(xb + 16));
                p1 = _mm256_fmadd_ps(_mm256_cvtepi32_ps(_mm256_cvtepi8_epi32(_mm_srli_si128(hi, 8))), _mm256_loadu_ps(xb + 24), p1);
                acc = _mm256_fmadd_ps(p0, _mm256_set1_ps(sc[0]), acc);
                acc = _mm256_fmadd_ps(p1, _mm256_set1_ps(sc[1]), acc);
                if (offset != 0.f) off += offset * xsum[size_t(b)];
            }
            result = hsum8(acc) + off;
        }
        y[r] = result;
    }
}

bool baseline_type(uint32_t t) { return t == TQO_IQ4_XS || t == TQO_IQ4_NL || t == TQO_Q4_K || t == TQO_IQ3_S || t == TQO_NVFP4G; }

// persistent workers woken by a generation counter (tests/bench_cpu_expert_mt.cpp:130-165); worker 0 is the caller
struct RowPool {
    std::vector<std::thread> th;
    std::atomic<long> gen{0};
    std::atomic<int> done{0};
    std::atomic<bool> stop{false};
    const std::function<void(int)> * work = nullptr;
    int n;
    explicit RowPool(int n_) : n(n_) {
        for (int i = 1; i < n; ++i) th.emplace_back([this, i]() {
            long seen = 0;
            for (;;) {
                const long g = gen.load(std::memory_order_acquire);
                if (g == seen) { if (stop.load(std::memory_order_acquire)) return; std::this_thread::yield(); continue; }
                seen = g;
                if (stop.load(std::memory_order_acquire)) return;
                (*work)(i);
                done.fetch_add(1, std::memory_order_release);
            }
        });
    }
    void run(const std::function<void(int)> & w) {
        work = &w;
        done.store(0, std::memory_order_release);
        gen.fetch_add(1, std::memory_order_release);
        w(0);
        while (done.load(std::memory_order_acquire) < n - 1) std::this_thread::yield();
    }
    ~RowPool() {
        stop.store(true, std::memory_order_release);
        gen.fetch_add(1, std::memory_order_release);
        for (auto & t : th) t.join();
    }
};

}  // namespace

int tqo_hardware_threads(void) { return int(std::thread::hardware_concurrency()); }

int tqo_cpu_matvec(uint32_t wtype, const void * W, int rows, int cols, const float * x, int mode, float * y) {
    int elems, bytes;
    if (!baseline_type(wtype) || !tqo_block_layout(wtype, &elems, &bytes) || cols % elems || cols % 32 || rows <= 0 || mode < 0 || mode > 2) return -1;
    XQ xq;
    if (mode) quant_x_blocks(x, cols, xq);
    matvec_rows(wtype, static_cast<const uint8_t *>(W), cols, x, mode ? &xq : nullptr, mode, 0, rows, y);
    return 0;
}

double tqo_cpu_expert_bench(uint32_t wtype, const void * gate, const void * up, const void * down, int hidden, int ff,
                            int n_expert, int threads, int int8_act, int reps, float * checksum) {
    int elems, bytes;
    if (!baseline_type(wtype) || !tqo_block_layout(wtype, &elems, &bytes) || hidden % elems || ff % elems || n_expert <= 0 || threads <= 0 || reps <= 0) return -1.0;
    const size_t stride = size_t(int64_t(ff) * hidden / elems) * bytes;
    const int mode = int8_act ? 1 : 0;
    std::vector<float> sums(static_cast<size_t>(n_expert), 0.f);
    auto pass = [&]() {
        std::atomic<int> next{0};
        auto worker = [&]() {
            std::vector<float> x(static_cast<size_t>(hidden), 0.5f), g(static_cast<size_t>(ff)), u(static_cast<size_t>(ff)), act(static_cast<size_t>(ff)), y(static_cast<size_t>(hidden));
            XQ xq, aq;
            for (;;) {
                const int e = next.fetch_add(1);
                if (e >= n_expert) break;
                for (int i = 0; i < hidden; ++i) x[size_t(i)] = 0.5f + 0.001f * float((i + e) & 15);
                if (int8_act) quant_x_blocks(x.data(), hidden, xq);
                matvec_rows(wtype, static_cast<const uint8_t *>(gate) + stride * e, hidden, x.data(), &xq, mode, 0, ff, g.data());
                matvec_rows(wtype, static_cast<const uint8_t *>(up) + stride * e, hidden, x.data(), &xq, mode, 0, ff, u.data());
                for (int o = 0; o < ff; ++o) act[size_t(o)] = (g[size_t(o)] / (1.f + std::exp(-g[size_t(o)]))) * u[size_t(o)];
                if (int8_act) quant_x_blocks(act.data(), ff, aq);
                matvec_rows(wtype, static_cast<const uint8_t *>(down) + stride * e, ff, act.data(), &aq, mode, 0, hidden, y.data());
                float s = 0.f;
                for (int i = 0; i < hidden; ++i) s += y[size_t(i)];
                sums[size_t(e)] = s;
            }
        };
        std::vector<std::thread> pool;
        for (int i = 1; i < threads; ++i) pool.emplace_back(worker);
        worker();
        for (auto & th : pool) th.join();
    };
    pass();
    const auto t0 = std::chrono::steady_clock::now();
    for (int r = 0; r < reps; ++r) pass();
    const auto t1 = std::chrono::steady_clock::now();
    if (checksum) { float s = 0.f; for (float v : sums) s += v; *checksum = s; }
    return std::chrono::duration<double>(t1 - t0).count() / reps;
}

double tqo_cpu_expert_latency(uint32_t wtype, const void * gate, const void * up, const void * down, int hidden, int ff,
                              int threads, int reps, float * checksum) {
    int elems, bytes;
    if (!baseline_type(wtype) || !tqo_block_layout(wtype, &elems, &bytes) || hidden % elems || ff % elems || threads <= 0 || reps <= 0) return -1.0;
    std::vector<float> x(static_cast<size_t>(hidden)), g(static_cast<size_t>(ff)), u(static_cast<size_t>(ff)), act(static_cast<size_t>(ff)), y(static_cast<size_t>(hidden));
    for (int i = 0; i < hidden; ++i) x[size_t(i)] = 0.5f + 0.001f * float(i & 15);
    XQ xq, aq;
    RowPool pool(threads);
    const std::function<void(int)> gate_up = [&](int t) {
        const int lo = int(int64_t(ff) * t / threads), hi = int(int64_t(ff) * (t + 1) / threads);
        matvec_rows(wtype, static_cast<const uint8_t *>(gate), hidden, x.data(), &xq, 1, lo, hi, g.data());
        matvec_rows(wtype, static_cast<const uint8_t *>(up), hidden, x.data(), &xq, 1, lo, hi, u.data());
    };
    const std::function<void(int)> down_rows = [&](int t) {
        const int lo = int(int64_t(hidden) * t / threads), hi = int(int64_t(hidden) * (t + 1) / threads);
        matvec_rows(wtype, static_cast<const uint8_t *>(down), ff, act.data(), &aq, 1, lo, hi, y.data());
    };
    auto expert = [&]() {   // the act row depends on every gate / up row: two phases, as the engine's miss pool runs them
        quant_x_blocks(x.data(), hidden, xq);
        pool.run(gate_up);
        for (int o = 0; o < ff; ++o) act[size_t(o)] = (g[size_t(o)] / (1.f + std::exp(-g[size_t(o)]))) * u[size_t(o)];
        quant_x_blocks(act.data(), ff, aq);
        pool.run(down_rows);
    };
    expert();
    const auto t0 = std::chrono::steady_clock::now();
    for (int r = 0; r < reps; ++r) expert();
    const auto t1 = std::chrono::steady_clock::now();
    if (checksum) { float s = 0.f; for (float v : y) s += v; *checksum = s; }
    return std::chrono::duration<double>(t1 - t0).count() / reps;
}

// The fp32 values of one sub-block (32 weights of a row) of a bank in the library's device layout, computed exactly as the
// reference's host decoder computes them (every product one correctly rounded fp32 multiply, in its order): shared by
// the fp32 dequantiser and the fp16 grouped products.
#pragma once
#include "formats.cuh"

namespace tqmoe {

__device__ __forceinline__ void decode_sub32(uint32_t type, const uint8_t * __restrict__ codes, const uint8_t * __restrict__ aux, int64_t rows_total, int cols,
                                             int64_t row, int s, float * __restrict__ y) {
    const int S = cols / 32, ib = s & 7;
    const uint8_t * cd = codes + (row * S + s) * code_bytes_per_sub(type);
    switch (type) {
        case TQMOE_IQ4_XS: {
            const uint2 rec = *reinterpret_cast<const uint2 *>(aux + iq4xs_aux_offset(row, S, s / 8));
            const float dl = __fmul_rn(half_bits_to_float(iq4xs_d_bits(rec)), float(iq4xs_lsm32(rec, ib)));
            const uint4 c = *reinterpret_cast<const uint4 *>(codes + iq4xs_code_offset(row, S, s));
            const uint32_t w[4] = {c.x, c.y, c.z, c.w};
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                uint32_t lo, hi;
                lookup16<kIq4T0, kIq4T1, kIq4T2, kIq4T3>(w[q], lo, hi);
#pragma unroll
                for (int b = 0; b < 4; ++b) {
                    y[4 * q + b] = __fmul_rn(dl, float(int8_t(lo >> (8 * b))));
                    y[16 + 4 * q + b] = __fmul_rn(dl, float(int8_t(hi >> (8 * b))));
                }
            }
            break;
        }
        case TQMOE_Q4_K: {
            const uint4 rec = *reinterpret_cast<const uint4 *>(aux + (row * (S / 8) + s / 8) * 16);
            const uint32_t sc12[3] = {rec.y, rec.z, rec.w};
            int sc, mn;
            q4k_scale_min(sc12, ib, sc, mn);
            const float d1 = __fmul_rn(half_bits_to_float(uint16_t(rec.x & 0xFFFFu)), float(sc));
            const float m1 = __fmul_rn(half_bits_to_float(uint16_t(rec.x >> 16)), float(mn));
            const uint4 c = *reinterpret_cast<const uint4 *>(cd);
            const uint32_t w[4] = {c.x, c.y, c.z, c.w};
#pragma unroll
            for (int q = 0; q < 4; ++q)
#pragma unroll
                for (int b = 0; b < 4; ++b) {
                    const uint32_t byte = (w[q] >> (8 * b)) & 0xFFu;
                    y[4 * q + b] = __fsub_rn(__fmul_rn(d1, float(byte & 15u)), m1);
                    y[16 + 4 * q + b] = __fsub_rn(__fmul_rn(d1, float(byte >> 4)), m1);
                }
            break;
        }
        case TQMOE_IQ3_S: {
            const uint4 rec = *reinterpret_cast<const uint4 *>(aux + (row * (S / 8) + s / 8) * 16);
            // rec: d | qh[0..1] << 16, qh[2..5], qh[6..7] | scales[0..1] << 16, scales[2..3]
            const uint32_t qh = ib < 2 ? (rec.x >> (16 + 8 * ib)) & 0xFFu : ib < 6 ? (rec.y >> (8 * (ib - 2))) & 0xFFu : (rec.z >> (8 * (ib - 6))) & 0xFFu;
            const uint32_t scb = (ib >> 1) < 2 ? (rec.z >> (16 + 8 * (ib >> 1))) & 0xFFu : (rec.w >> (8 * ((ib >> 1) - 2))) & 0xFFu;
            const float db = __fmul_rn(half_bits_to_float(uint16_t(rec.x & 0xFFFFu)), float(1 + 2 * int((scb >> (4 * (ib & 1))) & 15u)));
            const uint32_t * c = reinterpret_cast<const uint32_t *>(cd);
            const uint32_t qs[2] = {c[0], c[1]}, sg = c[2];
#pragma unroll
            for (int w = 0; w < 8; ++w) {
                const uint32_t g = d_iq3s_grid.v[((qs[w >> 2] >> (8 * (w & 3))) & 0xFFu) | (((qh >> w) & 1u) << 8)];
                const uint32_t sn = sg >> (4 * w);
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const float mag = __fmul_rn(db, float((g >> (8 * j)) & 0xFFu));
                    y[4 * w + j] = ((sn >> j) & 1u) ? -mag : mag;
                }
            }
            break;
        }
        case TQMOE_IQ3_XXS: {  // dequant.cpp:157-174: ((d * (0.5 + s)) * 0.5) * magnitude, sign applied last
            const float d = half_bits_to_float(*reinterpret_cast<const uint16_t *>(aux + (row * (S / 8) + s / 8) * 16));
            const uint32_t * c = reinterpret_cast<const uint32_t *>(cd);
            const uint32_t qs[2] = {c[0], c[1]}, word = c[2];
            const float db = __fmul_rn(__fmul_rn(d, __fadd_rn(0.5f, float(word >> 28))), 0.5f);
#pragma unroll
            for (int w = 0; w < 8; ++w) {   // group l = w / 2 of eight weights, half h = w % 2
                const uint32_t g = d_iq3xxs_grid.v[(qs[w >> 2] >> (8 * (w & 3))) & 0xFFu];
                const uint32_t sn = iq3xxs_signs(word, w >> 1) >> (4 * (w & 1));
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const float mag = __fmul_rn(db, float((g >> (8 * j)) & 0xFFu));
                    y[4 * w + j] = ((sn >> j) & 1u) ? -mag : mag;
                }
            }
            break;
        }
        case TQMOE_IQ2_S: {  // dequant.cpp:271-287: ((d * (0.5 + nibble)) * 0.25) * magnitude, one nibble per 16 weights
            const float d = half_bits_to_float(*reinterpret_cast<const uint16_t *>(aux + (row * (S / 8) + s / 8) * 16));
            const uint32_t * c = reinterpret_cast<const uint32_t *>(cd);
            const uint32_t low = c[0], sg = c[1], qh = c[2] & 0xFFu, sc = (c[2] >> 8) & 0xFFu;
            const float db[2] = {__fmul_rn(__fmul_rn(d, __fadd_rn(0.5f, float(sc & 15u))), 0.25f), __fmul_rn(__fmul_rn(d, __fadd_rn(0.5f, float(sc >> 4))), 0.25f)};
#pragma unroll
            for (int l = 0; l < 4; ++l) {
                const uint32_t idx = iq2s_index(low, qh, l), sn = (sg >> (8 * l)) & 0xFFu;
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const float mag = __fmul_rn(db[l >> 1], float((d_iq2s_grid.v[2 * idx + (j >> 2)] >> (8 * (j & 3))) & 0xFFu));
                    y[8 * l + j] = ((sn >> j) & 1u) ? -mag : mag;
                }
            }
            break;
        }
        case TQMOE_IQ2_XXS: {  // dequant.cpp:233-249: ((d * (0.5 + s)) * 0.25) * magnitude, sign applied last
            const float d = half_bits_to_float(*reinterpret_cast<const uint16_t *>(aux + (row * (S / 8) + s / 8) * 16));
            const uint2 c = *reinterpret_cast<const uint2 *>(cd);
            const float db = __fmul_rn(__fmul_rn(d, __fadd_rn(0.5f, float(c.y >> 28))), 0.25f);
#pragma unroll
            for (int l = 0; l < 4; ++l) {
                const uint32_t idx = (c.x >> (8 * l)) & 0xFFu, sn = iq3xxs_signs(c.y, l);
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const float mag = __fmul_rn(db, float((d_iq2xxs_grid.v[2 * idx + (j >> 2)] >> (8 * (j & 3))) & 0xFFu));
                    y[8 * l + j] = ((sn >> j) & 1u) ? -mag : mag;
                }
            }
            break;
        }
        case TQMOE_IQ2_XS: {  // dequant.cpp:252-268: ((d * (0.5 + nibble)) * 0.25) * magnitude, one nibble per 16 weights
            const float d = half_bits_to_float(*reinterpret_cast<const uint16_t *>(aux + (row * (S / 8) + s / 8) * 16));
            const uint32_t * c = reinterpret_cast<const uint32_t *>(cd);
            const uint32_t q2[2] = {c[0], c[1]}, sc = c[2] & 0xFFu;
            const float db[2] = {__fmul_rn(__fmul_rn(d, __fadd_rn(0.5f, float(sc & 15u))), 0.25f), __fmul_rn(__fmul_rn(d, __fadd_rn(0.5f, float(sc >> 4))), 0.25f)};
#pragma unroll
            for (int l = 0; l < 4; ++l) {
                const uint32_t q = (q2[l >> 1] >> (16 * (l & 1))) & 0xFFFFu, idx = q & 511u, sn = signs8(q >> 9);
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const float mag = __fmul_rn(db[l >> 1], float((d_iq2xs_grid.v[2 * idx + (j >> 2)] >> (8 * (j & 3))) & 0xFFu));
                    y[8 * l + j] = ((sn >> j) & 1u) ? -mag : mag;
                }
            }
            break;
        }
        case TQMOE_Q3_K: {  // dequant.cpp:118-131: (d * sc) * (q - 4), q = two low bits | mask bit << 2, one int8 scale per 16 weights
            const uint8_t * a = aux + (row * (S / 8) + s / 8) * 32;
            const float d = half_bits_to_float(*reinterpret_cast<const uint16_t *>(a + 16));
            const float ds[2] = {__fmul_rn(d, float(int8_t(a[2 * ib]))), __fmul_rn(d, float(int8_t(a[2 * ib + 1])))};
            const uint32_t * c = reinterpret_cast<const uint32_t *>(cd);
            const uint32_t lo[2] = {c[0], c[1]}, hb = c[2];
#pragma unroll
            for (int j = 0; j < 32; ++j) {
                const int q = int(((lo[j >> 4] >> (2 * (j & 15))) & 3u) | (((hb >> j) & 1u) << 2)) - 4;
                y[j] = __fmul_rn(ds[j >> 4], float(q));
            }
            break;
        }
        case TQMOE_Q2_K: {  // dequant.cpp:289-310: (d * scale) * q - dmin * min, a (scale, min) byte per 16 weights
            const uint8_t * a = aux + (row * (S / 8) + s / 8) * 32;
            const uint32_t dm = *reinterpret_cast<const uint32_t *>(a + 16);
            const float d = half_bits_to_float(uint16_t(dm & 0xFFFFu)), dmin = half_bits_to_float(uint16_t(dm >> 16));
            const float dl[2] = {__fmul_rn(d, float(a[2 * ib] & 15)), __fmul_rn(d, float(a[2 * ib + 1] & 15))};
            const float ml[2] = {__fmul_rn(dmin, float(a[2 * ib] >> 4)), __fmul_rn(dmin, float(a[2 * ib + 1] >> 4))};
            const uint2 c = *reinterpret_cast<const uint2 *>(cd);
            const uint32_t lo[2] = {c.x, c.y};
#pragma unroll
            for (int j = 0; j < 32; ++j) y[j] = __fsub_rn(__fmul_rn(dl[j >> 4], float((lo[j >> 4] >> (2 * (j & 15))) & 3u)), ml[j >> 4]);
            break;
        }
        case TQMOE_IQ1_S: {  // dequant.cpp:311-326: (d * (2 s + 1)) * (value + delta)
            const float d = half_bits_to_float(*reinterpret_cast<const uint16_t *>(aux + (row * (S / 8) + s / 8) * 16));
            const uint2 c = *reinterpret_cast<const uint2 *>(cd);
            const float dl = __fmul_rn(d, float(2 * int((c.y >> 12) & 7u) + 1)), delta = (c.y & 0x8000u) ? -0.125f : 0.125f;
#pragma unroll
            for (int l = 0; l < 4; ++l) {
                const uint32_t idx = ((c.x >> (8 * l)) & 0xFFu) | (((c.y >> (3 * l)) & 7u) << 8);
#pragma unroll
                for (int j = 0; j < 8; ++j)
                    y[8 * l + j] = __fmul_rn(dl, __fadd_rn(float(int8_t((d_iq1s_grid.v[2 * idx + (j >> 2)] >> (8 * (j & 3))) & 0xFFu)), delta));
            }
            break;
        }
        case TQMOE_Q4_0: {  // dequant.cpp:480-491: (q - 8) * d
            const float d = half_bits_to_float(*reinterpret_cast<const uint16_t *>(aux + (row * S + s) * 2));
            const uint4 c = *reinterpret_cast<const uint4 *>(cd);
            const uint32_t w[4] = {c.x, c.y, c.z, c.w};
#pragma unroll
            for (int q = 0; q < 4; ++q)
#pragma unroll
                for (int b = 0; b < 4; ++b) {
                    const uint32_t byte = (w[q] >> (8 * b)) & 0xFFu;
                    y[4 * q + b] = __fmul_rn(float(int(byte & 15u) - 8), d);
                    y[16 + 4 * q + b] = __fmul_rn(float(int(byte >> 4) - 8), d);
                }
            break;
        }
        case TQMOE_Q5_K: {  // dequant.cpp:102-116: (d * sc) * v - dmin * m, v = nibble + 16 * high bit
            const uint8_t * a = aux + (row * (S / 8) + s / 8) * 48;
            const uint4 rec = *reinterpret_cast<const uint4 *>(a);
            const uint32_t hb = *reinterpret_cast<const uint32_t *>(a + 16 + 4 * ib);
            const uint32_t sc12[3] = {rec.y, rec.z, rec.w};
            int sc, mn;
            q4k_scale_min(sc12, ib, sc, mn);
            const float d1 = __fmul_rn(half_bits_to_float(uint16_t(rec.x & 0xFFFFu)), float(sc));
            const float m1 = __fmul_rn(half_bits_to_float(uint16_t(rec.x >> 16)), float(mn));
            const uint4 c = *reinterpret_cast<const uint4 *>(cd);
            const uint32_t w[4] = {c.x, c.y, c.z, c.w};
#pragma unroll
            for (int q = 0; q < 4; ++q)
#pragma unroll
                for (int b = 0; b < 4; ++b) {
                    const uint32_t byte = (w[q] >> (8 * b)) & 0xFFu;
                    const int j = 4 * q + b;
                    y[j] = __fsub_rn(__fmul_rn(d1, float((byte & 15u) + 16u * ((hb >> j) & 1u))), m1);
                    y[16 + j] = __fsub_rn(__fmul_rn(d1, float((byte >> 4) + 16u * ((hb >> (16 + j)) & 1u))), m1);
                }
            break;
        }
        case TQMOE_Q6_K: {  // dequant.cpp:194-208: (d * sc) * (q - 32), one int8 scale per 16 weights
            const uint8_t * a = aux + (row * (S / 8) + s / 8) * 32;
            const float d = half_bits_to_float(*reinterpret_cast<const uint16_t *>(a + 16));
            const float d0 = __fmul_rn(d, float(int8_t(a[2 * ib]))), d1 = __fmul_rn(d, float(int8_t(a[2 * ib + 1])));
            const uint2 c0 = *reinterpret_cast<const uint2 *>(cd), c1 = *reinterpret_cast<const uint2 *>(cd + 8), hi = *reinterpret_cast<const uint2 *>(cd + 16);
            const uint32_t w[4] = {c0.x, c0.y, c1.x, c1.y};
            const uint32_t h2[2] = {hi.x, hi.y};
#pragma unroll
            for (int q = 0; q < 4; ++q)
#pragma unroll
                for (int b = 0; b < 4; ++b) {
                    const uint32_t byte = (w[q] >> (8 * b)) & 0xFFu;
                    const int j = 4 * q + b;
                    const int lo = int((byte & 15u) | (((h2[0] >> (2 * j)) & 3u) << 4)) - 32;
                    const int up = int((byte >> 4) | (((h2[1] >> (2 * j)) & 3u) << 4)) - 32;
                    y[j] = __fmul_rn(d0, float(lo));
                    y[16 + j] = __fmul_rn(d1, float(up));
                }
            break;
        }
        case TQMOE_IQ4_NL: {  // dequant.cpp:351-360: d * kv[q]
            const float d = half_bits_to_float(*reinterpret_cast<const uint16_t *>(aux + (row * S + s) * 2));
            const uint4 c = *reinterpret_cast<const uint4 *>(cd);
            const uint32_t w[4] = {c.x, c.y, c.z, c.w};
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                uint32_t lo, hi;
                lookup16<kIq4T0, kIq4T1, kIq4T2, kIq4T3>(w[q], lo, hi);
#pragma unroll
                for (int b = 0; b < 4; ++b) {
                    y[4 * q + b] = __fmul_rn(d, float(int8_t(lo >> (8 * b))));
                    y[16 + 4 * q + b] = __fmul_rn(d, float(int8_t(hi >> (8 * b))));
                }
            }
            break;
        }
        case TQMOE_Q8_0: {  // dequant.cpp:555-562: d * q
            const float d = half_bits_to_float(*reinterpret_cast<const uint16_t *>(aux + (row * S + s) * 2));
            const uint32_t * c = reinterpret_cast<const uint32_t *>(cd);
#pragma unroll
            for (int q = 0; q < 8; ++q) {
                const uint32_t w = c[q];
#pragma unroll
                for (int b = 0; b < 4; ++b) y[4 * q + b] = __fmul_rn(d, float(int8_t(w >> (8 * b))));
            }
            break;
        }
        case TQMOE_NVFP4G: {
            const float g = *reinterpret_cast<const float *>(aux + nvfp4_global_offset(rows_total, cols) + row * 4);
            const uint8_t * sc = aux + row * (cols / 16) + 2 * s;
            const float d0 = __fmul_rn(e4m3_to_float(sc[0]), g), d1 = __fmul_rn(e4m3_to_float(sc[1]), g);
            const uint4 c = *reinterpret_cast<const uint4 *>(cd);
            const uint32_t w[4] = {c.x, c.y, c.z, c.w};
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                uint32_t lo, hi;
                lookup16<kFp4T0, kFp4T1, kFp4T2, kFp4T3>(w[q], lo, hi);
#pragma unroll
                for (int b = 0; b < 4; ++b) {
                    // table holds twice the E2M1 value; halving is exact. -0 codes give -0 * d on the host: keep the sign
                    const uint32_t nlo = (w[q] >> (8 * b)) & 15u, nhi = (w[q] >> (8 * b + 4)) & 15u;
                    const float vlo = nlo == 8 ? -0.f : 0.5f * float(int8_t(lo >> (8 * b)));
                    const float vhi = nhi == 8 ? -0.f : 0.5f * float(int8_t(hi >> (8 * b)));
                    y[4 * q + b] = __fmul_rn(vlo, d0);
                    y[16 + 4 * q + b] = __fmul_rn(vhi, d1);
                }
            }
            break;
        }
    }

}

}  // namespace tqmoe

// Expert banks: GGUF block stream -> device layout (one thread per 32-weight sub-block), and the fp32 dequantiser
// whose values are those of the host decoder bit for bit (no fused multiply-add, same evaluation order).
#include "decode_sub.cuh"

namespace tqmoe {
namespace {

__device__ __forceinline__ uint32_t rd_u16(const uint8_t * p) { return uint32_t(p[0]) | uint32_t(p[1]) << 8; }
__device__ __forceinline__ uint32_t rd_u32(const uint8_t * p) { return rd_u16(p) | rd_u16(p + 2) << 16; }

// canonical nibble order of a sub-block: byte j = code of weight j | code of weight j + 16 << 4
template <class F> __device__ __forceinline__ void pack_sub(uint8_t * dst, F code) {
    uint32_t w[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        w[q] = 0;
#pragma unroll
        for (int b = 0; b < 4; ++b) { const int j = 4 * q + b; w[q] |= (uint32_t(code(j)) | uint32_t(code(j + 16)) << 4) << (8 * b); }
    }
    *reinterpret_cast<uint4 *>(dst) = make_uint4(w[0], w[1], w[2], w[3]);
}

__global__ __launch_bounds__(256) void load_k(uint32_t type, const uint8_t * __restrict__ src, int64_t rows_total, int cols,
                                              uint8_t * __restrict__ codes, uint8_t * __restrict__ aux, int * __restrict__ status) {
    const int S = cols / 32;
    const int64_t idx = int64_t(blockIdx.x) * 256 + threadIdx.x;
    if (idx >= rows_total * S) return;
    const int64_t row = idx / S;
    const int s = int(idx % S);
    uint8_t * cd = codes + idx * code_bytes_per_sub(type);
    switch (type) {
        case TQMOE_IQ4_XS: {  // 136 B per 256: d, scales_h, scales_l[4], qs[128]; nibble order already canonical; tile-major
            const uint8_t * blk = src + (row * (S / 8) + s / 8) * 136;
            const uint8_t * q = blk + 8 + 16 * (s & 7);
            pack_sub(codes + iq4xs_code_offset(row, S, s), [&](int j) { return j < 16 ? q[j] & 15 : q[j - 16] >> 4; });
            if ((s & 7) == 0) {
                uint8_t * a = aux + iq4xs_aux_offset(row, S, s / 8);
                const uint32_t head = rd_u32(blk);
                *reinterpret_cast<uint2 *>(a) = iq4xs_pack_rec(head & 0xFFFFu, head >> 16, rd_u32(blk + 4));
            }
            break;
        }
        case TQMOE_Q4_K: {  // 144 B per 256: d, dmin, scales[12], qs[128]; 64-weight chunk c: low nibbles then high
            const uint8_t * blk = src + (row * (S / 8) + s / 8) * 144;
            const int ib = s & 7;
            const uint8_t * q = blk + 16 + 32 * (ib >> 1);
            pack_sub(cd, [&](int j) { return (ib & 1) ? q[j] >> 4 : q[j] & 15; });
            if (ib == 0) {
                uint8_t * a = aux + (row * (S / 8) + s / 8) * 16;
                *reinterpret_cast<uint4 *>(a) = make_uint4(rd_u32(blk), rd_u32(blk + 4), rd_u32(blk + 8), rd_u32(blk + 12));
            }
            break;
        }
        case TQMOE_IQ3_S: {  // 110 B per 256: d, qs[64], qh[8], signs[32], scales[4]
            const uint8_t * blk = src + (row * (S / 8) + s / 8) * 110;
            const int ib = s & 7;
            uint32_t * o = reinterpret_cast<uint32_t *>(cd);
            o[0] = rd_u32(blk + 2 + 8 * ib);
            o[1] = rd_u32(blk + 2 + 8 * ib + 4);
            o[2] = rd_u32(blk + 74 + 4 * ib);
            if (ib == 0) {
                uint8_t * a = aux + (row * (S / 8) + s / 8) * 16;
                *reinterpret_cast<uint4 *>(a) = make_uint4(rd_u16(blk) | rd_u16(blk + 66) << 16, rd_u32(blk + 68),
                                                           rd_u16(blk + 72) | rd_u16(blk + 106) << 16, rd_u16(blk + 108));
            }
            break;
        }
        case TQMOE_IQ3_XXS: {  // 98 B per 256: d, qs[64] (lattice indices), 8 words of 4 x 7 sign bits + 4-bit scale
            const uint8_t * blk = src + (row * (S / 8) + s / 8) * 98;
            const int ib = s & 7;
            uint32_t * o = reinterpret_cast<uint32_t *>(cd);
            o[0] = rd_u32(blk + 2 + 8 * ib);
            o[1] = rd_u32(blk + 2 + 8 * ib + 4);
            o[2] = rd_u32(blk + 66 + 4 * ib);
            if (ib == 0) *reinterpret_cast<uint4 *>(aux + (row * (S / 8) + s / 8) * 16) = make_uint4(rd_u16(blk), 0, 0, 0);
            break;
        }
        case TQMOE_IQ2_S: {  // 82 B per 256: d, qs[32] (low index bytes), signs[32], qh[8], scales[8]
            const uint8_t * blk = src + (row * (S / 8) + s / 8) * 82;
            const int ib = s & 7;
            uint32_t * o = reinterpret_cast<uint32_t *>(cd);
            o[0] = rd_u32(blk + 2 + 4 * ib);
            o[1] = rd_u32(blk + 34 + 4 * ib);
            o[2] = uint32_t(blk[66 + ib]) | uint32_t(blk[74 + ib]) << 8;
            if (ib == 0) *reinterpret_cast<uint4 *>(aux + (row * (S / 8) + s / 8) * 16) = make_uint4(rd_u16(blk), 0, 0, 0);
            break;
        }
        case TQMOE_IQ2_XXS: {  // 66 B per 256: d, per sub-block four lattice index bytes and a word of 4 x 7 sign bits + 4-bit scale
            const uint8_t * blk = src + (row * (S / 8) + s / 8) * 66;
            const int ib = s & 7;
            *reinterpret_cast<uint2 *>(cd) = make_uint2(rd_u32(blk + 2 + 8 * ib), rd_u32(blk + 2 + 8 * ib + 4));
            if (ib == 0) *reinterpret_cast<uint4 *>(aux + (row * (S / 8) + s / 8) * 16) = make_uint4(rd_u16(blk), 0, 0, 0);
            break;
        }
        case TQMOE_IQ2_XS: {  // 74 B per 256: d, 32 x (9-bit lattice index | 7 sign bits << 9), scales[8] (a nibble per 16 weights)
            const uint8_t * blk = src + (row * (S / 8) + s / 8) * 74;
            const int ib = s & 7;
            uint32_t * o = reinterpret_cast<uint32_t *>(cd);
            o[0] = rd_u32(blk + 2 + 8 * ib);
            o[1] = rd_u32(blk + 2 + 8 * ib + 4);
            o[2] = blk[66 + ib];
            if (ib == 0) *reinterpret_cast<uint4 *>(aux + (row * (S / 8) + s / 8) * 16) = make_uint4(rd_u16(blk), 0, 0, 0);
            break;
        }
        case TQMOE_Q3_K: {  // 110 B per 256: hmask[32], qs[64], scales[12], d; sub-block i = 4 n + j holds weights 128 n + 32 j ..
            const uint8_t * blk = src + (row * (S / 8) + s / 8) * 110;
            const int ib = s & 7, n = ib >> 2, j = ib & 3;
            const uint8_t * qs = blk + 32 + 32 * n;
            uint32_t lo[2] = {0, 0}, hb = 0;   // two low bits per weight (byte k = weights 4 k .. 4 k + 3), the third bit per weight
#pragma unroll
            for (int l = 0; l < 32; ++l) {
                lo[l >> 4] |= uint32_t((qs[l] >> (2 * j)) & 3) << (2 * (l & 15));
                hb |= uint32_t((blk[l] >> ib) & 1) << l;
            }
            uint32_t * o = reinterpret_cast<uint32_t *>(cd);
            o[0] = lo[0]; o[1] = lo[1]; o[2] = hb;
            if (ib == 0) {   // the sixteen 6-bit scales, stored minus 32 as int8 (what the decoder multiplies by), then d
                const uint8_t * p = blk + 96;
                uint32_t w[4] = {0, 0, 0, 0};
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const uint32_t l4 = i < 8 ? p[i] & 15u : uint32_t(p[i - 8]) >> 4;
                    const uint32_t h2 = (uint32_t(p[8 + (i & 3)]) >> (2 * (i >> 2))) & 3u;
                    w[i >> 2] |= (((l4 | h2 << 4) - 32u) & 0xFFu) << (8 * (i & 3));
                }
                uint8_t * a = aux + (row * (S / 8) + s / 8) * 32;
                *reinterpret_cast<uint4 *>(a) = make_uint4(w[0], w[1], w[2], w[3]);
                *reinterpret_cast<uint4 *>(a + 16) = make_uint4(rd_u16(blk + 108), 0, 0, 0);
            }
            break;
        }
        case TQMOE_Q2_K: {  // 84 B per 256: scales[16] (scale | min << 4), qs[64], d, dmin; sub-block i = 4 n + j holds weights 128 n + 32 j ..
            const uint8_t * blk = src + (row * (S / 8) + s / 8) * 84;
            const int ib = s & 7, n = ib >> 2, j = ib & 3;
            const uint8_t * qs = blk + 16 + 32 * n;
            uint32_t lo[2] = {0, 0};   // two bits per weight, byte k = weights 4 k .. 4 k + 3
#pragma unroll
            for (int l = 0; l < 32; ++l) lo[l >> 4] |= uint32_t((qs[l] >> (2 * j)) & 3) << (2 * (l & 15));
            *reinterpret_cast<uint2 *>(cd) = make_uint2(lo[0], lo[1]);
            if (ib == 0) {
                uint8_t * a = aux + (row * (S / 8) + s / 8) * 32;
                *reinterpret_cast<uint4 *>(a) = make_uint4(rd_u32(blk), rd_u32(blk + 4), rd_u32(blk + 8), rd_u32(blk + 12));
                *reinterpret_cast<uint4 *>(a + 16) = make_uint4(rd_u32(blk + 80), 0, 0, 0);
            }
            break;
        }
        case TQMOE_IQ1_S: {  // 50 B per 256: d, qs[32] (low index bytes), qh[8] (4 x 3 index bits, 3-bit scale, delta sign)
            const uint8_t * blk = src + (row * (S / 8) + s / 8) * 50;
            const int ib = s & 7;
            *reinterpret_cast<uint2 *>(cd) = make_uint2(rd_u32(blk + 2 + 4 * ib), rd_u16(blk + 34 + 2 * ib));
            if (ib == 0) *reinterpret_cast<uint4 *>(aux + (row * (S / 8) + s / 8) * 16) = make_uint4(rd_u16(blk), 0, 0, 0);
            break;
        }
        case TQMOE_Q4_0: {  // 18 B per 32: d, qs[16] (byte j = weight j | weight j + 16 << 4: the canonical order)
            const uint8_t * blk = src + (row * S + s) * 18;
            pack_sub(cd, [&](int j) { return j < 16 ? blk[2 + j] & 15 : blk[2 + j - 16] >> 4; });
            *reinterpret_cast<uint16_t *>(aux + (row * S + s) * 2) = uint16_t(rd_u16(blk));
            break;
        }
        case TQMOE_Q5_K: {  // 176 B per 256: d, dmin, scales[12], qh[32] (bit j of byte l: weight l of sub-block j), qs[128] as Q4_K
            const uint8_t * blk = src + (row * (S / 8) + s / 8) * 176;
            const int ib = s & 7;
            const uint8_t * q = blk + 48 + 32 * (ib >> 1);
            pack_sub(cd, [&](int j) { return (ib & 1) ? q[j] >> 4 : q[j] & 15; });
            uint8_t * a = aux + (row * (S / 8) + s / 8) * 48;
            uint32_t hb = 0;
#pragma unroll
            for (int l = 0; l < 32; ++l) hb |= uint32_t((blk[16 + l] >> ib) & 1) << l;
            *reinterpret_cast<uint32_t *>(a + 16 + 4 * ib) = hb;
            if (ib == 0) *reinterpret_cast<uint4 *>(a) = make_uint4(rd_u32(blk), rd_u32(blk + 4), rd_u32(blk + 8), rd_u32(blk + 12));
            break;
        }
        case TQMOE_Q6_K: {  // 210 B per 256: ql[128], qh[64], scales[16], d; sub-block i = 4 n + j holds weights 128 n + 32 j ..
            const uint8_t * blk = src + (row * (S / 8) + s / 8) * 210;
            const int ib = s & 7, n = ib >> 2, j = ib & 3;
            const uint8_t * ql = blk + 64 * n + 32 * (j & 1), * qh = blk + 128 + 32 * n;
            __attribute__((aligned(16))) uint8_t low[16];   // 24-byte code records are 8-byte aligned: stored as three 8-byte pieces
            pack_sub(low, [&](int l) { return (j & 2) ? ql[l] >> 4 : ql[l] & 15; });
            reinterpret_cast<uint2 *>(cd)[0] = reinterpret_cast<const uint2 *>(low)[0];
            reinterpret_cast<uint2 *>(cd)[1] = reinterpret_cast<const uint2 *>(low)[1];
            uint32_t hi[2] = {0, 0};   // two bits per weight, byte k = weights 4 k .. 4 k + 3
#pragma unroll
            for (int l = 0; l < 32; ++l) hi[l >> 4] |= uint32_t((qh[l] >> (2 * j)) & 3) << (2 * (l & 15));
            *reinterpret_cast<uint2 *>(cd + 16) = make_uint2(hi[0], hi[1]);
            if (ib == 0) {
                uint8_t * a = aux + (row * (S / 8) + s / 8) * 32;
                *reinterpret_cast<uint4 *>(a) = make_uint4(rd_u32(blk + 192), rd_u32(blk + 196), rd_u32(blk + 200), rd_u32(blk + 204));
                *reinterpret_cast<uint4 *>(a + 16) = make_uint4(rd_u16(blk + 208), 0, 0, 0);
            }
            break;
        }
        case TQMOE_IQ4_NL: {  // 18 B per 32: d, qs[16] (byte j = weight j | weight j + 16 << 4: the canonical order)
            const uint8_t * blk = src + (row * S + s) * 18;
            pack_sub(cd, [&](int j) { return j < 16 ? blk[2 + j] & 15 : blk[2 + j - 16] >> 4; });
            *reinterpret_cast<uint16_t *>(aux + (row * S + s) * 2) = uint16_t(rd_u16(blk));
            break;
        }
        case TQMOE_Q8_0: {  // 34 B per 32: d, 32 int8
            const uint8_t * blk = src + (row * S + s) * 34;
            uint32_t * o = reinterpret_cast<uint32_t *>(cd);
#pragma unroll
            for (int q = 0; q < 8; ++q) o[q] = rd_u16(blk + 2 + 4 * q) | rd_u16(blk + 4 + 4 * q) << 16;
            *reinterpret_cast<uint16_t *>(aux + (row * S + s) * 2) = uint16_t(rd_u16(blk));
            break;
        }
        case TQMOE_NVFP4G: {  // 76 B per 128: global f32, 8 E4M3 scales, 64 code bytes (byte i of a 16-group: weights 2i, 2i + 1)
            const uint8_t * blk = src + (row * (S / 4) + s / 4) * 76;
            const int q4 = s & 3;
            const uint8_t * q = blk + 12 + 16 * q4;  // two 16-groups
            pack_sub(cd, [&](int j) { const uint8_t b = q[8 * (j >> 4) + ((j & 15) >> 1)]; return (j & 1) ? b >> 4 : b & 15; });
            uint8_t * a = aux + row * (cols / 16) + 2 * s;
            a[0] = blk[4 + 2 * q4];
            a[1] = blk[4 + 2 * q4 + 1];
            const uint32_t g = rd_u32(blk), g0 = rd_u32(src + row * (S / 4) * 76);
            if (g != g0 && status) atomicOr(status, 1);  // the row's blocks disagree on the global scale
            if (s == 0) *reinterpret_cast<uint32_t *>(aux + nvfp4_global_offset(rows_total, cols) + row * 4) = g0;
            break;
        }
    }
}

// fp32 values of one sub-block, written exactly as the host decoder computes them
__global__ __launch_bounds__(256) void dequant_k(uint32_t type, const uint8_t * __restrict__ codes, const uint8_t * __restrict__ aux,
                                                 int64_t rows_total, int cols, int64_t row0, int64_t nrows, float * __restrict__ out) {
    const int S = cols / 32;
    const int64_t idx = int64_t(blockIdx.x) * 256 + threadIdx.x;
    if (idx >= nrows * S) return;
    float y[32];
    decode_sub32(type, codes, aux, rows_total, cols, row0 + idx / S, int(idx % S), y);
    float4 * o = reinterpret_cast<float4 *>(out + idx * 32);
#pragma unroll
    for (int q = 0; q < 8; ++q) o[q] = make_float4(y[4 * q], y[4 * q + 1], y[4 * q + 2], y[4 * q + 3]);
}

}  // namespace

int32_t check_bank(const tqmoe_bank * b, const char * what, tqmoe_error * err) {
    if (!b || b->struct_size < sizeof(tqmoe_bank)) return fail(err, TQMOE_E_ARG, "%s: bank descriptor missing or too small", what);
    if (!is_bank_type(b->type)) return fail(err, TQMOE_E_UNSUPPORTED, "%s: bank type %u is not supported", what, b->type);
    if (!b->codes || !b->aux || b->experts <= 0 || b->rows <= 0 || b->cols <= 0) return fail(err, TQMOE_E_ARG, "%s: invalid bank shape or pointer", what);
    if (b->cols % (b->type == TQMOE_NVFP4G ? 128 : 256)) return fail(err, TQMOE_E_ARG, "%s: cols %d is not a multiple of the block size", what, b->cols);
    if (b->type == TQMOE_IQ4_XS && b->rows % 32) return fail(err, TQMOE_E_ARG, "%s: IQ4_XS banks need rows that are a multiple of 32 (got %d)", what, b->rows);
    return 0;
}

}  // namespace tqmoe

using namespace tqmoe;

extern "C" int32_t tqmoe_bank_layout(uint32_t type, int64_t rows_total, int32_t cols, size_t * code_bytes, size_t * aux_bytes, tqmoe_error * err) {
    if (!is_bank_type(type)) return fail(err, TQMOE_E_UNSUPPORTED, "tqmoe_bank_layout: bank type %u is not supported", type);
    if (rows_total <= 0 || cols <= 0 || cols % (type == TQMOE_NVFP4G ? 128 : 256)) return fail(err, TQMOE_E_ARG, "tqmoe_bank_layout: invalid shape");
    if (type == TQMOE_IQ4_XS && rows_total % 32) return fail(err, TQMOE_E_ARG, "tqmoe_bank_layout: IQ4_XS banks need a multiple of 32 rows");
    if (code_bytes) *code_bytes = size_t(rows_total * code_row_bytes(type, cols));
    if (aux_bytes) *aux_bytes = type == TQMOE_NVFP4G ? size_t(nvfp4_global_offset(rows_total, cols) + rows_total * 4) : size_t(rows_total * aux_row_bytes(type, cols));
    return ok(err);
}

extern "C" int32_t tqmoe_bank_load(uint32_t type, const void * gguf_blocks, int64_t rows_total, int32_t cols, void * codes, void * aux,
                                   int32_t * status, void * stream, tqmoe_error * err) {
    if (int32_t rc = tqmoe_bank_layout(type, rows_total, cols, nullptr, nullptr, err)) return rc;
    if (!gguf_blocks || !codes || !aux) return fail(err, TQMOE_E_ARG, "tqmoe_bank_load: null pointer");
    if (int32_t rc = need_device(err, "tqmoe_bank_load")) return rc;
    const int64_t subs = rows_total * (cols / 32);
    if ((subs + 255) / 256 > 0x7FFFFFFF) return fail(err, TQMOE_E_ARG, "tqmoe_bank_load: bank too large for one call");
    load_k<<<unsigned((subs + 255) / 256), 256, 0, static_cast<hipStream_t>(stream)>>>(type, static_cast<const uint8_t *>(gguf_blocks), rows_total, cols,
                                                                                      static_cast<uint8_t *>(codes), static_cast<uint8_t *>(aux), status);
    return launched(err, "tqmoe_bank_load");
}

extern "C" int32_t tqmoe_bank_dequant(const tqmoe_bank * bank, int64_t row0, int64_t nrows, float * out, void * stream, tqmoe_error * err) {
    if (int32_t rc = check_bank(bank, "tqmoe_bank_dequant", err)) return rc;
    const int64_t rows_total = int64_t(bank->experts) * bank->rows;
    if (!out || row0 < 0 || nrows <= 0 || row0 + nrows > rows_total) return fail(err, TQMOE_E_ARG, "tqmoe_bank_dequant: invalid row range");
    if (int32_t rc = need_device(err, "tqmoe_bank_dequant")) return rc;
    const int64_t subs = nrows * (bank->cols / 32);
    if ((subs + 255) / 256 > 0x7FFFFFFF) return fail(err, TQMOE_E_ARG, "tqmoe_bank_dequant: range too large for one call");
    dequant_k<<<unsigned((subs + 255) / 256), 256, 0, static_cast<hipStream_t>(stream)>>>(bank->type, static_cast<const uint8_t *>(bank->codes),
                                                                                         static_cast<const uint8_t *>(bank->aux), rows_total, bank->cols, row0, nrows, out);
    return launched(err, "tqmoe_bank_dequant");
}

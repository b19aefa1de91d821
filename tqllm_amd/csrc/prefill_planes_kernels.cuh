// Prefill-sized expert products on the matrix pipe with 8-bit operands: grouped int8 x int8 -> int32 GEMMs for IQ4_XS,
// IQ3_S and Q4_K banks (exact weights), and an fp8 x fp8 -> fp32 GEMM for NVFP4G banks (weights widened to E4M3).
//
// Operands. Activations are 8 bits per input row with one fp32 scale per row: int8 (amax / 127) or E4M3 (amax / 448). The
// rows of every expert's assignments are gathered into tiles of 32 rows, experts in order, each expert padded to whole
// tiles, and stored operand-major: the 1 KB that the 64 lanes of a wave feed to one v_mfma_i32_32x32x32_i8 as operand A
// (lane = 32 g + r holds, for row r and 32-weight sub-block j, the 16 values {8g..8g+7} and {16+8g..16+8g+7} in the byte
// order of the bank's code bytes) is contiguous, sub-blocks in order. A wave then loads its operand with one fully
// coalesced instruction and no shuffle. The two 8-byte halves of that operand are the operands of two
// v_mfma_f32_32x32x16_fp8_fp8, and two sub-blocks' 32 bytes the operand of one
// v_mfma_f32_32x32x64_f8f6f4 (which is what the fp8 path issues), so the fp8 path shares the layout.
// Integer weights stay exact. A value is d * p with an integer p per weight of up to 13 bits (IQ4_XS: (ls - 32) * kv[q];
// IQ3_S: (1 + 2 ls) * (+-lattice magnitude); Q4_K: sc * q, with the minimum's coefficient mn as a further plane that
// is constant over a sub-block). p is split as 64 * h + l with h, l int8, taken per sub-block from 16-entry lookup
// tables in LDS (one pair per scale value) and applied with v_perm_b32. The planes go through one MFMA each that
// accumulate over the whole 256-weight super-block, so the scales cost no vector instruction per product; per
// super-block the results fold as acc += d * (64 * acc_h + acc_l) - dmin * acc_m in fp32.
// With a scale per row and 32-value sub-block in place of one per row (the reference's other int8 mode) the integer sums
// cannot ride through the super-block: every sub-block's MFMAs start from zero and its sums are scaled by the weights'
// scale and the row's scale of that sub-block as they join the fp32 result (the BLK instances of the kernel).
// NVFP4G weights are e2m1 * E4M3 scale (per 16 weights) * fp32 global (per row): the product of the first two is rounded
// to E4M3 (a declared lossy operand: six significant bits into four), again through a 16-entry table per scale byte; the
// fp8 MFMA accumulates in fp32 over the whole row and the global multiplies the result.
//
// Blocks. A work item is one expert, a chunk of up to kChunkTiles row tiles of its assignments and one unit of weight
// rows: 32 rows of both banks (gate / up, SwiGLU fused) or 64 rows of one bank (down). Resident blocks of eight waves
// take items from counters (one per XCD, so that a chunk's rows stay in one L2). Per super-block the waves decode the
// unit's weights once into a double-buffered LDS stage that every wave then reads as operand B (decoding super-block
// i + 1 overlaps the products of super-block i, one barrier per super-block); a wave multiplies one row tile with the
// weights of both operand slots, so a loaded piece of operand A (prefetched into registers a few k-steps ahead) serves
// every product with it and SwiGLU pairs values the same lane holds. A chunk of a single row tile has nothing to share:
// every wave then takes the tile against 32 weight rows of its own (four units per item), decoding straight into
// registers with no barrier in the loop.
#pragma once
#include "act_image.cuh"
#include "decode_api.cuh"
#include "formats.cuh"

#include <algorithm>
#include <type_traits>

namespace tqmoe {

// (types that cross translation units)
// Index of the grouped rows, kept behind the row scales: tile_base[e] = row tiles of the experts before e
// (tiles_e = ceil(count_e / 32)), chunk_base[e] = chunks of kChunkTiles row tiles before e, chunk_base2[e] = chunks of twice
// as many, all with a total at [experts].
// Behind them 16 counters the product kernel hands work out with (zero between launches).
constexpr int kPlanCounters = 16;
struct Plan { const int * tile_base, * chunk_base, * chunk_base2; int * counters; };
__host__ __device__ inline Plan plan_at(const float * scale, int64_t grouped_rows, int experts) {
    const int * p = reinterpret_cast<const int *>(scale + grouped_rows);
    return Plan{p, p + experts + 1, p + 2 * (experts + 1), const_cast<int *>(p) + 3 * (experts + 1)};
}

struct GemmArgs {
    BankView b0, b1;          // gate and up; down: the same bank twice
    const int8_t * xq;        // grouped operand-major row tiles
    const float * xs;         // [row tiles * 32]
    const int * counts;       // [experts]
    const int * offsets;      // [experts + 1]
    const int * perm;         // assignment indices grouped by expert
    Plan plan;
    int experts;
    uint16_t * out;           // fp16 [assignments][rows]: silu(gate) * up, or the plain product
    int units;                // weight-row units per expert: rows / 32 (gate / up, and down with NB = 1), rows / 64 (down, NB = 2)
    int unit_group;           // consecutive units an item runs through (a divisor of units): short rows get more per item
    int shared_expert;        // index of the expert whose rows (gate / up) or columns (down) stop at shared_lim, or -1
    int shared_lim;
    const float * xbs;        // a scale per row and 32-value sub-block, [row tile][sub-block][32 rows] (the rows' own scales are then 1), or null
    Glu glu;                  // gate / up: the optional clamp of the SwiGLU inputs
    int out_bf16;             // the results as bf16 rows in place of fp16
};

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kChunkTiles = 8;                // row tiles (of 32 assignments) per chunk; formats with registers to spare take chunks of twice that
constexpr int kPlanExperts = 1024;              // experts whose index a block keeps in LDS

// four scaled values -> four operand bytes: int8 (round to nearest) or E4M3 (round to nearest even; the values are
// clamped to +-448 first, so the conversion never leaves the finite codes)
template <bool F8> __device__ __forceinline__ uint32_t pack4_q(float a, float b, float c, float d) {
    if constexpr (F8) {
        auto clamp = [](float v) { return fminf(fmaxf(v, -448.f), 448.f); };
        int w = __builtin_amdgcn_cvt_pk_fp8_f32(clamp(a), clamp(b), 0, false);
        w = __builtin_amdgcn_cvt_pk_fp8_f32(clamp(c), clamp(d), w, true);
        return uint32_t(w);
    } else {
        return uint32_t(__float2int_rn(a) & 0xFF) | uint32_t(__float2int_rn(b) & 0xFF) << 8 | uint32_t(__float2int_rn(c) & 0xFF) << 16 |
               uint32_t(__float2int_rn(d) & 0xFF) << 24;
    }
}
template <bool F8> constexpr float kOperandMax = F8 ? 448.f : 127.f;

// largest e in [0, experts) with base[e] <= unit, for unit < base[experts] (experts with no unit share their successor's
// base and are skipped by taking the last of equal entries)
__device__ __forceinline__ int owner_of(const int * __restrict__ base, int experts, int unit) {
    int lo = 0, hi = experts;            // base[lo] <= unit < base[hi]
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (base[mid] <= unit) lo = mid; else hi = mid;
    }
    return lo;
}

typedef float v16f __attribute__((ext_vector_type(16)));
typedef int v2i __attribute__((ext_vector_type(2)));

// four codes (bytes of idx3: index within a table half; sel: position + 4 * half) through a 16-entry byte table
__device__ __forceinline__ int pick16(uint4 t, uint32_t idx3, uint32_t sel) {
    return int(__builtin_amdgcn_perm(__builtin_amdgcn_perm(t.w, t.z, idx3), __builtin_amdgcn_perm(t.y, t.x, idx3), sel));
}
// the eight 4-bit codes of a dword as lookup keys: low nibbles (weights j) and high nibbles (weights j + 16)
struct NibbleKeys { uint32_t i_lo, s_lo, i_hi, s_hi; };
__device__ __forceinline__ NibbleKeys nibble_keys(uint32_t c) {
    return NibbleKeys{c & 0x07070707u, ((c >> 1) & 0x04040404u) | 0x03020100u, (c >> 4) & 0x07070707u, ((c >> 5) & 0x04040404u) | 0x03020100u};
}
// 16 codes (two dwords) through the two 16-entry tables of their sub-block scale: h and l planes, 16 int8 each, in operand
// order (values 8g.., 16 + 8g.., 8g + 4.., 16 + 8g + 4..)
__device__ __forceinline__ void decode_planes(uint2 c, uint4 th, uint4 tl, v4i & h, v4i & l) {
    const uint32_t cw[2] = {c.x, c.y};
#pragma unroll
    for (int w = 0; w < 2; ++w) {
        const NibbleKeys k = nibble_keys(cw[w]);
        h[2 * w] = pick16(th, k.i_lo, k.s_lo);
        h[2 * w + 1] = pick16(th, k.i_hi, k.s_hi);
        l[2 * w] = pick16(tl, k.i_lo, k.s_lo);
        l[2 * w + 1] = pick16(tl, k.i_hi, k.s_hi);
    }
}
// an integer of up to 13 bits as 64 * hi + lo with lo in [-32, 32) and both in int8
__device__ __forceinline__ void split_planes(int v, uint8_t & hi, uint8_t & lo) {
    const int l = ((v + 32) & 63) - 32;
    lo = uint8_t(l);
    hi = uint8_t((v - l) >> 6);
}

// The two ways through the kernel (a lone row tile, a shared chunk) must give a row the same bits: the fold of a
// super-block and the epilogue are spelled with explicitly rounded operations, and the product that is converted to fp16
// passes through an opaque register, so that no path turns multiply + convert into one mixed-precision instruction
// (one rounding instead of two: different bits at ties).
__device__ __forceinline__ float fold_sb(float acc, int h, int l, float d) { return __fmaf_rn(float((h << 6) + l), d, acc); }
__device__ __forceinline__ uint16_t to_half_bits(float v) {
    asm volatile("" : "+v"(v));
    return __half_as_ushort(__float2half_rn(v));
}
__device__ __forceinline__ uint16_t swiglu_half(float g_acc, float u_acc, float sc, const Glu glu) {
    float gv = __fmul_rn(g_acc, sc), uv = __fmul_rn(u_acc, sc);
    glu_clamp_inputs(glu, gv, uv);
    const float den = __fadd_rn(1.f, __expf(-gv));
    return to_half_bits(__fmul_rn(glu_clamp_silu(glu, __fdiv_rn(gv, den)), uv));
}
__device__ __forceinline__ uint16_t scaled_half(float acc, float sc, int bf16) {
    const float v = __fmul_rn(acc, sc);
    return bf16 ? float_to_bf16_bits(v) : to_half_bits(v);
}

__device__ const int8_t kIq4Values[16] = {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113};

// ------------------------------------------------------------------------------------------------ bank formats
// What the kernel needs of a format. Lane (n, g) of a wave holds, of weight row n of a 32-row tile and one sub-block, the
// 16 weights {8g..8g+7} and {16+8g..16+8g+7}: Src are its base pointers, Code what it loads per sub-block, Rec what
// decoding needs of the sub-block's super-block, DRec what the fold needs of it (the lane's row, any g).
// planes() turns a Code into kPlanes operand registers; tables() fills the lookup tables (and the lattice) in LDS.
struct WIq4xs {   // tile-major codes (512 B per sub-block of a tile), 8-byte records (256 B per super-block of a tile)
    static constexpr bool kFoldSub = false;     // one scale per 32 weights: every sub-block's product is folded on its own
    static constexpr bool kWideChunks = false;   // chunks of sixteen row tiles on eight waves (two row tiles a wave)
    static constexpr int kPlanes = 2, kTabBytes = 64 * 32, kLattice = 1;
    static constexpr bool kFp8 = false, kMin = false, kRowMul = false;
    struct Code { uint2 c; };
    typedef uint2 Rec;
    typedef uint2 DRec;
    struct Src { const uint8_t * codes, * aux; };
    static __device__ __forceinline__ void tables(uint8_t * tab, uint32_t *, int tid, int threads) {   // per 6-bit scale: 16 h bytes, 16 l bytes
        for (int i = tid; i < 64 * 16; i += threads) split_planes(int(kIq4Values[i & 15]) * ((i >> 4) - 32), tab[(i >> 4) * 32 + (i & 15)], tab[(i >> 4) * 32 + 16 + (i & 15)]);
    }
    static __device__ __forceinline__ Src src(const BankView & b, int e, int wtile, int n, int g) {
        const int S = b.cols / 32;
        const int64_t tile_g = int64_t(e) * (b.rows / 32) + wtile;
        return Src{b.codes + tile_g * S * 512 + n * 16 + g * 8, b.aux + tile_g * (S / 8) * 256 + n * 8};
    }
    static __device__ __forceinline__ Code code(const Src & s, int sub) { return Code{*reinterpret_cast<const uint2 *>(s.codes + int64_t(sub) * 512)}; }
    static __device__ __forceinline__ Rec rec(const Src & s, int sb) { return *reinterpret_cast<const uint2 *>(s.aux + int64_t(sb) * 256); }
    static __device__ __forceinline__ DRec drec(const Src & s, int sb) { return rec(s, sb); }
    static __device__ __forceinline__ void planes(const Code & c, const Rec & r, int ib, int, const uint8_t * tab, const uint32_t *, v4i * p) {
        const uint4 * t = reinterpret_cast<const uint4 *>(tab + iq4xs_ls(r, ib) * 32);
        decode_planes(c.c, t[0], t[1], p[0], p[1]);
    }
    static __device__ __forceinline__ float d(const DRec & r) { return half_bits_to_float(iq4xs_d_bits(r)); }
    static __device__ __forceinline__ float dmin(const DRec &) { return 0.f; }
    static __device__ __forceinline__ float rowmul(const BankView &, int, int, int) { return 1.f; }
};

// IQ4_XS for rows with a scale per sub-block: the sub-block scale no longer needs to ride inside the operand (every
// sub-block's sums are scaled on their own anyway), so one plane of the 16 table values and d * (ls - 32) as the
// sub-block's fp32 scale: half the MFMAs, LDS traffic and lookups of the two-plane form.
struct WIq4xsSub : WIq4xs {
    static constexpr bool kFoldSub = true;
    static constexpr int kPlanes = 1, kTabBytes = 16;
    static __device__ __forceinline__ void tables(uint8_t *, uint32_t *, int, int) {}
    static __device__ __forceinline__ void planes(const Code & c, const Rec &, int, int, const uint8_t *, const uint32_t *, v4i * p) {
        uint32_t lo, hi;
        lookup16<kIq4T0, kIq4T1, kIq4T2, kIq4T3>(c.c.x, lo, hi);
        p[0][0] = int(lo); p[0][1] = int(hi);
        lookup16<kIq4T0, kIq4T1, kIq4T2, kIq4T3>(c.c.y, lo, hi);
        p[0][2] = int(lo); p[0][3] = int(hi);
    }
    static __device__ __forceinline__ float d_sub(const DRec & r, int ib) {   // exact: an 11-bit significand times a 6-bit integer
        return __fmul_rn(half_bits_to_float(iq4xs_d_bits(r)), float(iq4xs_lsm32(r, ib)));
    }
};

struct WQ4k {   // row-major: 16 code bytes per sub-block, a 16-byte record (d | dmin << 16, twelve bytes of 6-bit scales and minimums) per super-block
    static constexpr bool kFoldSub = false;     // one scale per 32 weights: every sub-block's product is folded on its own
    static constexpr bool kWideChunks = false;   // chunks of sixteen row tiles on eight waves (two row tiles a wave)
    static constexpr int kPlanes = 3, kTabBytes = 64 * 32, kLattice = 1;
    static constexpr bool kFp8 = false, kMin = true, kRowMul = false;
    struct Code { uint2 c; };
    typedef uint4 Rec;
    typedef uint32_t DRec;
    struct Src { const uint8_t * codes, * aux; };
    static __device__ __forceinline__ void tables(uint8_t * tab, uint32_t *, int tid, int threads) {   // per 6-bit scale sc: sc * q for the 16 codes
        for (int i = tid; i < 64 * 16; i += threads) split_planes((i & 15) * (i >> 4), tab[(i >> 4) * 32 + (i & 15)], tab[(i >> 4) * 32 + 16 + (i & 15)]);
    }
    static __device__ __forceinline__ Src src(const BankView & b, int e, int wtile, int n, int g) {
        const int S = b.cols / 32;
        const int64_t row = int64_t(e) * b.rows + wtile * 32 + n;
        return Src{b.codes + row * S * 16 + g * 8, b.aux + row * (S / 8) * 16};
    }
    static __device__ __forceinline__ Code code(const Src & s, int sub) { return Code{*reinterpret_cast<const uint2 *>(s.codes + int64_t(sub) * 16)}; }
    static __device__ __forceinline__ Rec rec(const Src & s, int sb) { return *reinterpret_cast<const uint4 *>(s.aux + int64_t(sb) * 16); }
    static __device__ __forceinline__ DRec drec(const Src & s, int sb) { return *reinterpret_cast<const uint32_t *>(s.aux + int64_t(sb) * 16); }
    static __device__ __forceinline__ void planes(const Code & c, const Rec & r, int ib, int, const uint8_t * tab, const uint32_t *, v4i * p) {
        int sc, mn;
        q4k_scale_min_flat(r.y, r.z, r.w, ib, sc, mn);
        const uint4 * t = reinterpret_cast<const uint4 *>(tab + sc * 32);
        decode_planes(c.c, t[0], t[1], p[0], p[1]);
        const int m = mn * 0x01010101;   // the minimum's coefficient, the same for the sub-block's 32 weights
        p[2] = v4i{m, m, m, m};
    }
    static __device__ __forceinline__ float d(const DRec & r) { return half_bits_to_float(uint16_t(r & 0xFFFFu)); }
    static __device__ __forceinline__ float dmin(const DRec & r) { return half_bits_to_float(uint16_t(r >> 16)); }
    static __device__ __forceinline__ float rowmul(const BankView &, int, int, int) { return 1.f; }
};

// Q4_K for rows with a scale per sub-block, likewise: the 4-bit codes themselves as one plane (no lookup), a plane of ones
// whose product is the sum of the row's values, and d * sc, dmin * mn as the sub-block's fp32 scales.
struct WQ4kSub : WQ4k {
    static constexpr bool kFoldSub = true;
    static constexpr int kPlanes = 2, kTabBytes = 16;
    typedef uint4 DRec;      // the whole record: the fold needs the sub-block's scale and minimum
    static __device__ __forceinline__ void tables(uint8_t *, uint32_t *, int, int) {}
    static __device__ __forceinline__ DRec drec(const Src & s, int sb) { return rec(s, sb); }
    static __device__ __forceinline__ void planes(const Code & c, const Rec &, int, int, const uint8_t *, const uint32_t *, v4i * p) {
        p[0] = v4i{int(c.c.x & 0x0F0F0F0Fu), int((c.c.x >> 4) & 0x0F0F0F0Fu), int(c.c.y & 0x0F0F0F0Fu), int((c.c.y >> 4) & 0x0F0F0F0Fu)};
        p[1] = v4i{0x01010101, 0x01010101, 0x01010101, 0x01010101};
    }
    static __device__ __forceinline__ float d_sub(const DRec & r, int ib) {      // exact: 11 bits times 6 bits
        int sc, mn;
        q4k_scale_min_flat(r.y, r.z, r.w, ib, sc, mn);
        return __fmul_rn(half_bits_to_float(uint16_t(r.x & 0xFFFFu)), float(sc));
    }
    static __device__ __forceinline__ float dmin_sub(const DRec & r, int ib) {
        int sc, mn;
        q4k_scale_min_flat(r.y, r.z, r.w, ib, sc, mn);
        return __fmul_rn(half_bits_to_float(uint16_t(r.x >> 16)), float(mn));
    }
};

struct WIq3s {   // row-major: 12 code bytes per sub-block (8 lattice indices, 32 sign bits), a 16-byte record per super-block
    static constexpr bool kFoldSub = false;     // one scale per 32 weights: every sub-block's product is folded on its own
    static constexpr bool kWideChunks = false;   // chunks of sixteen row tiles on eight waves (two row tiles a wave)
    static constexpr int kPlanes = 2, kTabBytes = 16 * 32, kLattice = 512;
    static constexpr bool kFp8 = false, kMin = false, kRowMul = false;
    struct Code { uint32_t qs0, qs1, sg; };
    typedef uint4 Rec;       // d | qh[0..1] << 16, qh[2..5], qh[6..7] | scales[0..1] << 16, scales[2..3]
    typedef uint32_t DRec;
    struct Src { const uint8_t * codes, * aux; };
    // per 4-bit scale ls the 16 products (1 + 2 ls) * (+-(2 j + 1)): code = sign << 3 | magnitude index j
    static __device__ __forceinline__ void tables(uint8_t * tab, uint32_t * lat, int tid, int threads) {
        for (int i = tid; i < 16 * 16; i += threads) {
            const int mag = (1 + 2 * (i >> 4)) * (2 * (i & 7) + 1);
            split_planes((i & 8) ? -mag : mag, tab[(i >> 4) * 32 + (i & 15)], tab[(i >> 4) * 32 + 16 + (i & 15)]);
        }
        for (int i = tid; i < 512; i += threads) lat[i] = d_iq3s_grid.v[i];
    }
    static __device__ __forceinline__ Src src(const BankView & b, int e, int wtile, int n, int) {
        const int S = b.cols / 32;
        const int64_t row = int64_t(e) * b.rows + wtile * 32 + n;
        return Src{b.codes + row * S * 12, b.aux + row * (S / 8) * 16};
    }
    static __device__ __forceinline__ Code code(const Src & s, int sub) {
        const uint32_t * c = reinterpret_cast<const uint32_t *>(s.codes + int64_t(sub) * 12);
        return Code{c[0], c[1], c[2]};
    }
    static __device__ __forceinline__ Rec rec(const Src & s, int sb) { return *reinterpret_cast<const uint4 *>(s.aux + int64_t(sb) * 16); }
    static __device__ __forceinline__ DRec drec(const Src & s, int sb) { return *reinterpret_cast<const uint32_t *>(s.aux + int64_t(sb) * 16); }
    static __device__ __forceinline__ void planes(const Code & c, const Rec & r, int ib, int g, const uint8_t * tab, const uint32_t * lat, v4i * p) {
        const uint32_t qh = ib < 2 ? (r.x >> (16 + 8 * ib)) & 0xFFu : ib < 6 ? (r.y >> (8 * (ib - 2))) & 0xFFu : (r.z >> (8 * (ib - 6))) & 0xFFu;
        const uint32_t scb = (ib >> 1) < 2 ? (r.z >> (16 + 8 * (ib >> 1))) & 0xFFu : (r.w >> (8 * ((ib >> 1) - 2))) & 0xFFu;
        const uint4 * t = reinterpret_cast<const uint4 *>(tab + ((scb >> (4 * (ib & 1))) & 15u) * 32);
        const uint4 th = t[0], tl = t[1];
#pragma unroll
        for (int q = 0; q < 4; ++q) {   // operand dword q = the group of four weights 2 g + q / 2 (+ 4 for odd q)
            const int w = 2 * g + (q >> 1) + 4 * (q & 1);
            const uint32_t idx = (((w < 4 ? c.qs0 : c.qs1) >> (8 * (w & 3))) & 0xFFu) | (((qh >> w) & 1u) << 8);
            const uint32_t mag = lat[idx];                                      // bytes 1, 3, .., 15
            const uint32_t i3 = (mag >> 1) & 0x07070707u, sel = (spread4(c.sg >> (4 * w)) << 2) | 0x03020100u;
            p[0][q] = pick16(th, i3, sel);
            p[1][q] = pick16(tl, i3, sel);
        }
    }
    static __device__ __forceinline__ float d(const DRec & r) { return half_bits_to_float(uint16_t(r & 0xFFFFu)); }
    static __device__ __forceinline__ float dmin(const DRec &) { return 0.f; }
    static __device__ __forceinline__ float rowmul(const BankView &, int, int, int) { return 1.f; }
};

// ---- the other lattice formats of the reference's MMQ list: magnitudes of 4 or 8 weights per lattice point (LDS copy of the
// lattice), a sign bit per weight, a 4-bit scale s with multiplier 2 s + 1 per sub-block or per 16 weights, one fp16 d per
// super-block (first dword of a 16-byte record). p = (2 s + 1) * (+-magnitude) through 16-entry tables per scale:
// code = sign << 3 | level index of the magnitude (magnitude >> SH). value = d * p / 4 (IQ3_XXS) or d * p / 8 (IQ2).
template <int SH> __device__ __forceinline__ void lattice_planes(uint32_t mag, uint32_t sign4, uint4 th, uint4 tl, v4i * p, int q) {
    const uint32_t i3 = (mag >> SH) & 0x07070707u, sel = (spread4(sign4) << 2) | 0x03020100u;
    p[0][q] = pick16(th, i3, sel);
    p[1][q] = pick16(tl, i3, sel);
}
template <class LEVEL> __device__ __forceinline__ void lattice_tables(uint8_t * tab, int tid, int threads, LEVEL level) {
    for (int i = tid; i < 16 * 16; i += threads) {
        const int mag = (1 + 2 * (i >> 4)) * level(i & 7);
        split_planes((i & 8) ? -mag : mag, tab[(i >> 4) * 32 + (i & 15)], tab[(i >> 4) * 32 + 16 + (i & 15)]);
    }
}
struct WLatticeBase {   // row-major, a 16-byte record per super-block whose first 16 bits are d
    static constexpr int kPlanes = 2, kTabBytes = 16 * 32;
    static constexpr bool kFp8 = false, kMin = false, kRowMul = false, kWideChunks = false, kFoldSub = false;
    typedef uint32_t Rec;    // unused by the decode (the scales sit in the code bytes)
    typedef uint32_t DRec;
    struct Src { const uint8_t * codes, * aux; };
    template <int CB> static __device__ __forceinline__ Src src_of(const BankView & b, int e, int wtile, int n) {
        const int S = b.cols / 32;
        const int64_t row = int64_t(e) * b.rows + wtile * 32 + n;
        return Src{b.codes + row * S * CB, b.aux + row * (S / 8) * 16};
    }
    static __device__ __forceinline__ Rec rec(const Src &, int) { return 0; }
    static __device__ __forceinline__ DRec drec(const Src & s, int sb) { return *reinterpret_cast<const uint32_t *>(s.aux + int64_t(sb) * 16); }
    static __device__ __forceinline__ float dmin(const DRec &) { return 0.f; }
    static __device__ __forceinline__ float rowmul(const BankView &, int, int, int) { return 1.f; }
};

struct WIq3xxs : WLatticeBase {   // 12 code bytes: 8 lattice indices (4 weights each), a word of 4 x 7 sign bits + the scale
    static constexpr int kLattice = 256;
    struct Code { uint32_t qs0, qs1, word; };
    static __device__ __forceinline__ void tables(uint8_t * tab, uint32_t * lat, int tid, int threads) {
        lattice_tables(tab, tid, threads, [](int l) { return int(iq3xxs_level(uint32_t(l))); });
        for (int i = tid; i < 256; i += threads) lat[i] = d_iq3xxs_grid.v[i];
    }
    static __device__ __forceinline__ Src src(const BankView & b, int e, int wtile, int n, int) { return src_of<12>(b, e, wtile, n); }
    static __device__ __forceinline__ Code code(const Src & s, int sub) {
        const uint32_t * c = reinterpret_cast<const uint32_t *>(s.codes + int64_t(sub) * 12);
        return Code{c[0], c[1], c[2]};
    }
    static __device__ __forceinline__ void planes(const Code & c, const Rec &, int, int g, const uint8_t * tab, const uint32_t * lat, v4i * p) {
        const uint4 * t = reinterpret_cast<const uint4 *>(tab + (c.word >> 28) * 32);
        const uint4 th = t[0], tl = t[1];
#pragma unroll
        for (int q = 0; q < 4; ++q) {   // operand dword q = the group of four weights w
            const int w = 2 * g + (q >> 1) + 4 * (q & 1);
            const uint32_t mag = lat[((w < 4 ? c.qs0 : c.qs1) >> (8 * (w & 3))) & 0xFFu];
            lattice_planes<3>(mag, iq3xxs_signs(c.word, w >> 1) >> (4 * (w & 1)), th, tl, p, q);
        }
    }
    static __device__ __forceinline__ float d(const DRec & r) { return half_bits_to_float(uint16_t(r & 0xFFFFu)) * 0.25f; }
};

__device__ __forceinline__ int iq2_level(int l) { return l == 0 ? 8 : l == 1 ? 25 : l == 2 ? 43 : 0; }

struct WIq2xxs : WLatticeBase {   // 8 code bytes: 4 lattice indices (8 weights each), a word of 4 x 7 sign bits + the scale
    static constexpr int kLattice = 512;
    struct Code { uint2 c; };
    static __device__ __forceinline__ void tables(uint8_t * tab, uint32_t * lat, int tid, int threads) {
        lattice_tables(tab, tid, threads, iq2_level);
        for (int i = tid; i < 512; i += threads) lat[i] = d_iq2xxs_grid.v[i];
    }
    static __device__ __forceinline__ Src src(const BankView & b, int e, int wtile, int n, int) { return src_of<8>(b, e, wtile, n); }
    static __device__ __forceinline__ Code code(const Src & s, int sub) { return Code{*reinterpret_cast<const uint2 *>(s.codes + int64_t(sub) * 8)}; }
    static __device__ __forceinline__ void planes(const Code & c, const Rec &, int, int g, const uint8_t * tab, const uint32_t * lat, v4i * p) {
        const uint4 * t = reinterpret_cast<const uint4 *>(tab + (c.c.y >> 28) * 32);
        const uint4 th = t[0], tl = t[1];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int w = 2 * g + (q >> 1) + 4 * (q & 1), l = w >> 1, half = w & 1;   // group of eight weights, its half
            const uint32_t mag = lat[2 * ((c.c.x >> (8 * l)) & 0xFFu) + half];
            lattice_planes<4>(mag, iq3xxs_signs(c.c.y, l) >> (4 * half), th, tl, p, q);
        }
    }
    static __device__ __forceinline__ float d(const DRec & r) { return half_bits_to_float(uint16_t(r & 0xFFFFu)) * 0.125f; }
};

struct WIq2xs : WLatticeBase {   // 12 code bytes: 4 x (9-bit lattice index | 7 sign bits << 9), a byte of two scales (a nibble per 16 weights)
    static constexpr int kLattice = 1024;
    struct Code { uint32_t q0, q1, sc; };
    static __device__ __forceinline__ void tables(uint8_t * tab, uint32_t * lat, int tid, int threads) {
        lattice_tables(tab, tid, threads, iq2_level);
        for (int i = tid; i < 1024; i += threads) lat[i] = d_iq2xs_grid.v[i];
    }
    static __device__ __forceinline__ Src src(const BankView & b, int e, int wtile, int n, int) { return src_of<12>(b, e, wtile, n); }
    static __device__ __forceinline__ Code code(const Src & s, int sub) {
        const uint32_t * c = reinterpret_cast<const uint32_t *>(s.codes + int64_t(sub) * 12);
        return Code{c[0], c[1], c[2]};
    }
    static __device__ __forceinline__ void planes(const Code & c, const Rec &, int, int g, const uint8_t * tab, const uint32_t * lat, v4i * p) {
        const uint4 * t0 = reinterpret_cast<const uint4 *>(tab + (c.sc & 15u) * 32), * t1 = reinterpret_cast<const uint4 *>(tab + ((c.sc >> 4) & 15u) * 32);
        const uint4 th[2] = {t0[0], t1[0]}, tl[2] = {t0[1], t1[1]};
#pragma unroll
        for (int q = 0; q < 4; ++q) {   // odd operand dwords hold weights 16..31: the second scale
            const int w = 2 * g + (q >> 1) + 4 * (q & 1), l = w >> 1, half = w & 1;
            const uint32_t qq = ((l < 2 ? c.q0 : c.q1) >> (16 * (l & 1))) & 0xFFFFu;
            const uint32_t mag = lat[2 * (qq & 511u) + half];
            lattice_planes<4>(mag, signs8(qq >> 9) >> (4 * half), th[q & 1], tl[q & 1], p, q);
        }
    }
    static __device__ __forceinline__ float d(const DRec & r) { return half_bits_to_float(uint16_t(r & 0xFFFFu)) * 0.125f; }
};

struct WIq2s : WLatticeBase {   // 12 code bytes: 4 low index bytes, 4 sign bytes, a byte of high index bits, a byte of two scales
    static constexpr int kLattice = 2048;
    struct Code { uint32_t low, sg, hs; };
    static __device__ __forceinline__ void tables(uint8_t * tab, uint32_t * lat, int tid, int threads) {
        lattice_tables(tab, tid, threads, iq2_level);
        for (int i = tid; i < 2048; i += threads) lat[i] = d_iq2s_grid.v[i];
    }
    static __device__ __forceinline__ Src src(const BankView & b, int e, int wtile, int n, int) { return src_of<12>(b, e, wtile, n); }
    static __device__ __forceinline__ Code code(const Src & s, int sub) {
        const uint32_t * c = reinterpret_cast<const uint32_t *>(s.codes + int64_t(sub) * 12);
        return Code{c[0], c[1], c[2]};
    }
    static __device__ __forceinline__ void planes(const Code & c, const Rec &, int, int g, const uint8_t * tab, const uint32_t * lat, v4i * p) {
        const uint32_t qh = c.hs & 0xFFu, sc = (c.hs >> 8) & 0xFFu;
        const uint4 * t0 = reinterpret_cast<const uint4 *>(tab + (sc & 15u) * 32), * t1 = reinterpret_cast<const uint4 *>(tab + (sc >> 4) * 32);
        const uint4 th[2] = {t0[0], t1[0]}, tl[2] = {t0[1], t1[1]};
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int w = 2 * g + (q >> 1) + 4 * (q & 1), l = w >> 1, half = w & 1;
            const uint32_t mag = lat[2 * iq2s_index(c.low, qh, l) + half];
            lattice_planes<4>(mag, ((c.sg >> (8 * l)) & 0xFFu) >> (4 * half), th[q & 1], tl[q & 1], p, q);
        }
    }
    static __device__ __forceinline__ float d(const DRec & r) { return half_bits_to_float(uint16_t(r & 0xFFFFu)) * 0.125f; }
};

struct WIq1s : WLatticeBase {   // 8 code bytes: 4 low index bytes (8 weights each), 16 bits of 4 x 3 high index bits, a 3-bit scale, the delta's sign
    // value = d * (2 s + 1) * (g +- 1/8), g in {-1, 0, 1}: p = (2 s + 1) * (8 g +- 1), |p| <= 135, value = d * p / 8; a table per
    // (scale, delta sign), code = the lattice byte's low two bits (0, 1, 3 for g = 0, 1, -1)
    static constexpr int kLattice = 4096;
    struct Code { uint2 c; };
    static __device__ __forceinline__ void tables(uint8_t * tab, uint32_t * lat, int tid, int threads) {
        for (int i = tid; i < 16 * 16; i += threads) {
            const int t = i >> 4, c = i & 15, gval = c == 1 ? 1 : c == 3 ? -1 : 0;
            split_planes((2 * (t & 7) + 1) * (8 * gval + ((t & 8) ? -1 : 1)), tab[t * 32 + c], tab[t * 32 + 16 + c]);
        }
        for (int i = tid; i < 4096; i += threads) lat[i] = d_iq1s_grid.v[i];
    }
    static __device__ __forceinline__ Src src(const BankView & b, int e, int wtile, int n, int) { return src_of<8>(b, e, wtile, n); }
    static __device__ __forceinline__ Code code(const Src & s, int sub) { return Code{*reinterpret_cast<const uint2 *>(s.codes + int64_t(sub) * 8)}; }
    static __device__ __forceinline__ void planes(const Code & c, const Rec &, int, int g, const uint8_t * tab, const uint32_t * lat, v4i * p) {
        const uint4 * t = reinterpret_cast<const uint4 *>(tab + (((c.c.y >> 12) & 7u) | ((c.c.y >> 12) & 8u)) * 32);
        const uint4 th = t[0], tl = t[1];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int w = 2 * g + (q >> 1) + 4 * (q & 1), l = w >> 1, half = w & 1;
            const uint32_t idx = ((c.c.x >> (8 * l)) & 0xFFu) | (((c.c.y >> (3 * l)) & 7u) << 8);
            const uint32_t i3 = lat[2 * idx + half] & 0x03030303u;
            p[0][q] = pick16(th, i3, 0x03020100u);
            p[1][q] = pick16(tl, i3, 0x03020100u);
        }
    }
    static __device__ __forceinline__ float d(const DRec & r) { return half_bits_to_float(uint16_t(r & 0xFFFFu)) * 0.125f; }
};

struct WIq4nl {   // row-major: 16 code bytes per sub-block (nibbles as IQ4_XS), one fp16 scale per 32 weights (eight per 256 in the aux plane)
    static constexpr int kPlanes = 1, kTabBytes = 16, kLattice = 1;
    static constexpr bool kFp8 = false, kMin = false, kRowMul = false, kWideChunks = false;
    static constexpr bool kFoldSub = true;
    struct Code { uint2 c; };
    typedef uint32_t Rec;    // unused by the decode
    typedef uint4 DRec;      // the eight scales of the row's super-block
    struct Src { const uint8_t * codes, * aux; };
    static __device__ __forceinline__ void tables(uint8_t *, uint32_t *, int, int) {}
    static __device__ __forceinline__ Src src(const BankView & b, int e, int wtile, int n, int g) {
        const int S = b.cols / 32;
        const int64_t row = int64_t(e) * b.rows + wtile * 32 + n;
        return Src{b.codes + row * S * 16 + g * 8, b.aux + row * S * 2};
    }
    static __device__ __forceinline__ Code code(const Src & s, int sub) { return Code{*reinterpret_cast<const uint2 *>(s.codes + int64_t(sub) * 16)}; }
    static __device__ __forceinline__ Rec rec(const Src &, int) { return 0; }
    static __device__ __forceinline__ DRec drec(const Src & s, int sb) { return *reinterpret_cast<const uint4 *>(s.aux + int64_t(sb) * 16); }
    static __device__ __forceinline__ void planes(const Code & c, const Rec &, int, int, const uint8_t *, const uint32_t *, v4i * p) {
        uint32_t lo, hi;
        lookup16<kIq4T0, kIq4T1, kIq4T2, kIq4T3>(c.c.x, lo, hi);
        p[0][0] = int(lo); p[0][1] = int(hi);
        lookup16<kIq4T0, kIq4T1, kIq4T2, kIq4T3>(c.c.y, lo, hi);
        p[0][2] = int(lo); p[0][3] = int(hi);
    }
    static __device__ __forceinline__ float d_sub(const DRec & r, int ib) {   // scale of sub-block ib of the super-block
        const uint32_t w = (ib >> 1) == 0 ? r.x : (ib >> 1) == 1 ? r.y : (ib >> 1) == 2 ? r.z : r.w;
        return half_bits_to_float(uint16_t((w >> (16 * (ib & 1))) & 0xFFFFu));
    }
    static __device__ __forceinline__ float d(const DRec &) { return 1.f; }
    static __device__ __forceinline__ float dmin(const DRec &) { return 0.f; }
    static __device__ __forceinline__ float rowmul(const BankView &, int, int, int) { return 1.f; }
};

// Q4_0: IQ4_NL's layout; the weight is the nibble minus 8 (no lookup)
struct WQ4_0 : WIq4nl {
    static __device__ __forceinline__ void planes(const Code & c, const Rec &, int, int, const uint8_t *, const uint32_t *, v4i * p) {
        p[0] = v4i{int(minus_k<8>(c.c.x & 0x0F0F0F0Fu)), int(minus_k<8>((c.c.x >> 4) & 0x0F0F0F0Fu)),
                   int(minus_k<8>(c.c.y & 0x0F0F0F0Fu)), int(minus_k<8>((c.c.y >> 4) & 0x0F0F0F0Fu))};
    }
};

// Q8_0: 32 int8 values per sub-block, the operand itself: lane (n, g) reads values 8g.. and 16 + 8g.. (two 8-byte loads)
struct WQ8_0 : WIq4nl {
    struct Code { uint2 lo, hi; };
    static __device__ __forceinline__ Src src(const BankView & b, int e, int wtile, int n, int g) {
        const int S = b.cols / 32;
        const int64_t row = int64_t(e) * b.rows + wtile * 32 + n;
        return Src{b.codes + row * S * 32 + g * 8, b.aux + row * S * 2};
    }
    static __device__ __forceinline__ Code code(const Src & s, int sub) {
        const uint8_t * c = s.codes + int64_t(sub) * 32;
        return Code{*reinterpret_cast<const uint2 *>(c), *reinterpret_cast<const uint2 *>(c + 16)};
    }
    static __device__ __forceinline__ void planes(const Code & c, const Rec &, int, int, const uint8_t *, const uint32_t *, v4i * p) {
        p[0] = v4i{int(c.lo.x), int(c.hi.x), int(c.lo.y), int(c.hi.y)};
    }
};

// Q5_K: Q4_K's layout and header, and a word per sub-block with the fifth bit of its 32 codes (after the header in the
// 48-byte record). The products sc * q of a 5-bit code q are looked up as for Q4_K, from two pairs of 16-entry tables per
// scale (q below 16, q from 16 on), and the fifth bit chooses between the two results bit by bit.
struct WQ5k {
    static constexpr bool kFoldSub = false, kWideChunks = false;
    static constexpr int kPlanes = 3, kTabBytes = 64 * 64, kLattice = 1;
    static constexpr bool kFp8 = false, kMin = true, kRowMul = false;
    struct Code { uint2 c; uint32_t hb; };
    typedef uint4 Rec;
    typedef uint32_t DRec;
    struct Src { const uint8_t * codes, * aux; };
    static __device__ __forceinline__ void tables(uint8_t * tab, uint32_t *, int tid, int threads) {   // per 6-bit scale sc: sc * q, q = 0..15 (h, l), q = 16..31 (h, l)
        for (int i = tid; i < 64 * 32; i += threads) {
            const int sc = i >> 5, q = i & 31;
            split_planes(q * sc, tab[sc * 64 + (q >> 4) * 32 + (q & 15)], tab[sc * 64 + (q >> 4) * 32 + 16 + (q & 15)]);
        }
    }
    static __device__ __forceinline__ Src src(const BankView & b, int e, int wtile, int n, int g) {
        const int S = b.cols / 32;
        const int64_t row = int64_t(e) * b.rows + wtile * 32 + n;
        return Src{b.codes + row * S * 16 + g * 8, b.aux + row * (S / 8) * 48};
    }
    static __device__ __forceinline__ Code code(const Src & s, int sub) {
        return Code{*reinterpret_cast<const uint2 *>(s.codes + int64_t(sub) * 16), *reinterpret_cast<const uint32_t *>(s.aux + int64_t(sub >> 3) * 48 + 16 + 4 * (sub & 7))};
    }
    static __device__ __forceinline__ Rec rec(const Src & s, int sb) { return *reinterpret_cast<const uint4 *>(s.aux + int64_t(sb) * 48); }
    static __device__ __forceinline__ DRec drec(const Src & s, int sb) { return *reinterpret_cast<const uint32_t *>(s.aux + int64_t(sb) * 48); }
    static __device__ __forceinline__ int choose(uint32_t mask, int on, int off) { return int((uint32_t(on) & mask) | (uint32_t(off) & ~mask)); }
    static __device__ __forceinline__ void planes(const Code & c, const Rec & r, int ib, int g, const uint8_t * tab, const uint32_t *, v4i * p) {
        int sc, mn;
        q4k_scale_min_flat(r.y, r.z, r.w, ib, sc, mn);
        const uint4 * t = reinterpret_cast<const uint4 *>(tab + sc * 64);
        const uint4 h0 = t[0], l0 = t[1], h1 = t[2], l1 = t[3];
        const uint32_t cw[2] = {c.c.x, c.c.y};
        const uint32_t hb = c.hb >> (8 * g);   // the fifth bits of the lane's values: bits 0..7 (values 8g..), 16..23 (values 16 + 8g..)
#pragma unroll
        for (int w = 0; w < 2; ++w) {
            const NibbleKeys k = nibble_keys(cw[w]);
            const uint32_t m_lo = spread4(hb >> (4 * w)) * 0xFFu, m_hi = spread4(hb >> (16 + 4 * w)) * 0xFFu;
            p[0][2 * w] = choose(m_lo, pick16(h1, k.i_lo, k.s_lo), pick16(h0, k.i_lo, k.s_lo));
            p[0][2 * w + 1] = choose(m_hi, pick16(h1, k.i_hi, k.s_hi), pick16(h0, k.i_hi, k.s_hi));
            p[1][2 * w] = choose(m_lo, pick16(l1, k.i_lo, k.s_lo), pick16(l0, k.i_lo, k.s_lo));
            p[1][2 * w + 1] = choose(m_hi, pick16(l1, k.i_hi, k.s_hi), pick16(l0, k.i_hi, k.s_hi));
        }
        const int m = mn * 0x01010101;
        p[2] = v4i{m, m, m, m};
    }
    static __device__ __forceinline__ float d(const DRec & r) { return half_bits_to_float(uint16_t(r & 0xFFFFu)); }
    static __device__ __forceinline__ float dmin(const DRec & r) { return half_bits_to_float(uint16_t(r >> 16)); }
    static __device__ __forceinline__ float rowmul(const BankView &, int, int, int) { return 1.f; }
};

// Q5_K for rows with a scale per sub-block: the 5-bit codes themselves as one plane, a plane of ones, d * sc and dmin * mn
// as the sub-block's fp32 scales (as WQ4kSub)
struct WQ5kSub : WQ5k {
    static constexpr bool kFoldSub = true;
    static constexpr int kPlanes = 2, kTabBytes = 16;
    typedef uint4 DRec;
    static __device__ __forceinline__ void tables(uint8_t *, uint32_t *, int, int) {}
    static __device__ __forceinline__ DRec drec(const Src & s, int sb) { return rec(s, sb); }
    static __device__ __forceinline__ void planes(const Code & c, const Rec &, int, int g, const uint8_t *, const uint32_t *, v4i * p) {
        const uint32_t hb = c.hb >> (8 * g);
        p[0] = v4i{int((c.c.x & 0x0F0F0F0Fu) | (spread4(hb) << 4)), int(((c.c.x >> 4) & 0x0F0F0F0Fu) | (spread4(hb >> 16) << 4)),
                   int((c.c.y & 0x0F0F0F0Fu) | (spread4(hb >> 4) << 4)), int(((c.c.y >> 4) & 0x0F0F0F0Fu) | (spread4(hb >> 20) << 4))};
        p[1] = v4i{0x01010101, 0x01010101, 0x01010101, 0x01010101};
    }
    static __device__ __forceinline__ float d_sub(const DRec & r, int ib) {      // exact: 11 bits times 6 bits
        int sc, mn;
        q4k_scale_min_flat(r.y, r.z, r.w, ib, sc, mn);
        return __fmul_rn(half_bits_to_float(uint16_t(r.x & 0xFFFFu)), float(sc));
    }
    static __device__ __forceinline__ float dmin_sub(const DRec & r, int ib) {
        int sc, mn;
        q4k_scale_min_flat(r.y, r.z, r.w, ib, sc, mn);
        return __fmul_rn(half_bits_to_float(uint16_t(r.x >> 16)), float(mn));
    }
};

struct WNvfp4 {   // row-major: 16 code bytes per sub-block, one E4M3 scale byte per 16 weights, one fp32 global per row
    static constexpr bool kFoldSub = false;     // one scale per 32 weights: every sub-block's product is folded on its own
    static constexpr bool kWideChunks = true;   // chunks of sixteen row tiles on eight waves (two row tiles a wave)
    static constexpr int kPlanes = 1, kTabBytes = 256 * 16, kLattice = 1;
    static constexpr bool kFp8 = true, kRowMul = true;
    struct Code { uint2 c; };
    typedef uint4 Rec;       // the 16 scale bytes of the row's super-block
    typedef uint32_t DRec;   // unused: nothing is folded
    struct Src { const uint8_t * codes, * aux; };
    // per scale byte the 16 products e2m1(code) * e4m3(scale) / 8, rounded to E4M3 (nearest even); the division keeps the
    // largest product (6 * 448) inside the format, and rowmul() gives the 8 back
    static __device__ __forceinline__ void tables(uint8_t * tab, uint32_t *, int tid, int threads) {
        uint32_t * t32 = reinterpret_cast<uint32_t *>(tab);
        for (int i = tid; i < 256 * 4; i += threads) {
            const float sc = e4m3_to_float(uint32_t(i >> 2));
            float v[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int c = 4 * (i & 3) + j;
                const uint32_t tb = ((c < 4 ? kFp4T0 : c < 8 ? kFp4T1 : c < 12 ? kFp4T2 : kFp4T3) >> (8 * (c & 3))) & 0xFFu;   // twice the e2m1 value
                v[j] = float(int8_t(tb)) * 0.0625f * sc;
            }
            t32[i] = pack4_q<true>(v[0], v[1], v[2], v[3]);
        }
    }
    static __device__ __forceinline__ Src src(const BankView & b, int e, int wtile, int n, int g) {
        const int S = b.cols / 32;
        const int64_t row = int64_t(e) * b.rows + wtile * 32 + n;
        return Src{b.codes + row * S * 16 + g * 8, b.aux + row * (b.cols / 16)};
    }
    static __device__ __forceinline__ Code code(const Src & s, int sub) { return Code{*reinterpret_cast<const uint2 *>(s.codes + int64_t(sub) * 16)}; }
    static __device__ __forceinline__ Rec rec(const Src & s, int sb) { return *reinterpret_cast<const uint4 *>(s.aux + int64_t(sb) * 16); }
    static __device__ __forceinline__ DRec drec(const Src &, int) { return 0; }
    static __device__ __forceinline__ void planes(const Code & c, const Rec & r, int ib, int, const uint8_t * tab, const uint32_t *, v4i * p) {
        const uint32_t pair = ((ib >> 1) == 0 ? r.x : (ib >> 1) == 1 ? r.y : (ib >> 1) == 2 ? r.z : r.w) >> (16 * (ib & 1));
        const uint4 t0 = *reinterpret_cast<const uint4 *>(tab + (pair & 0xFFu) * 16), t1 = *reinterpret_cast<const uint4 *>(tab + ((pair >> 8) & 0xFFu) * 16);
        const uint32_t cw[2] = {c.c.x, c.c.y};
#pragma unroll
        for (int w = 0; w < 2; ++w) {   // low nibbles: the sub-block's first 16 weights (first scale), high nibbles: the other 16
            const NibbleKeys k = nibble_keys(cw[w]);
            p[0][2 * w] = pick16(t0, k.i_lo, k.s_lo);
            p[0][2 * w + 1] = pick16(t1, k.i_hi, k.s_hi);
        }
    }
    static __device__ __forceinline__ float d(const DRec &) { return 1.f; }
    static __device__ __forceinline__ float dmin(const DRec &) { return 0.f; }
    static __device__ __forceinline__ float rowmul(const BankView & b, int e, int wtile, int n) {
        return 8.f * *reinterpret_cast<const float *>(b.aux + nvfp4_global_offset(b.rows_total, b.cols) + (int64_t(e) * b.rows + wtile * 32 + n) * 4);
    }
};

// one sub-block's products of a row tile with the planes of a weight tile
template <class W> struct Acc {
    v16i plane[W::kFp8 || W::kFoldSub ? 1 : W::kPlanes];   // int32 sums of the current super-block (unused by the fp8 path and by per-sub-block folds)
    v16f sum;                               // fp32 result so far
};
template <class W> __device__ __forceinline__ void acc_clear(Acc<W> & a) {
#pragma unroll
    for (int i = 0; i < 16; ++i) a.sum[i] = 0.f;
}
// two consecutive sub-blocks (64 weights of the rows) of operand A and of the weight planes. int8: one
// v_mfma_i32_32x32x32_i8 per sub-block and plane. fp8: one v_mfma_f32_32x32x64_f8f6f4 (both operands E4M3, no block
// scales) for the pair: twice the rate of the 32x32x16 fp8 instruction on this part.
typedef int v8i __attribute__((ext_vector_type(8)));
template <class W> __device__ __forceinline__ void acc_step2(Acc<W> & a, v4i x0, v4i x1, const v4i * w0, const v4i * w1, bool first_of_sb, const typename W::DRec & r,
                                                            int ib0) {
    if constexpr (W::kFp8) {
        const v8i x = {x0[0], x0[1], x0[2], x0[3], x1[0], x1[1], x1[2], x1[3]};
        const v8i w = {w0[0][0], w0[0][1], w0[0][2], w0[0][3], w1[0][0], w1[0][1], w1[0][2], w1[0][3]};
        a.sum = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(x, w, a.sum, 0, 0, 0, 0, 0, 0);
    } else if constexpr (W::kFoldSub) {   // a scale per sub-block: each sub-block's integer sums (exact) go into the fp32 result at once
        const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        const v16i s0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(x0, w0[0], zero, 0, 0, 0);
        const v16i s1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(x1, w1[0], zero, 0, 0, 0);
        const float d0 = W::d_sub(r, ib0), d1 = W::d_sub(r, ib0 + 1);
#pragma unroll
        for (int i = 0; i < 16; ++i) a.sum[i] = __fmaf_rn(float(s1[i]), d1, __fmaf_rn(float(s0[i]), d0, a.sum[i]));
        asm volatile("" : "+v"(a.sum));   // (pinned: see acc_step2_blocks)
    } else {
        const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
        for (int p = 0; p < W::kPlanes; ++p) a.plane[p] = __builtin_amdgcn_mfma_i32_32x32x32_i8(x0, w0[p], first_of_sb ? zero : a.plane[p], 0, 0, 0);
#pragma unroll
        for (int p = 0; p < W::kPlanes; ++p) a.plane[p] = __builtin_amdgcn_mfma_i32_32x32x32_i8(x1, w1[p], a.plane[p], 0, 0, 0);
    }
}
// One sub-block's product where the rows carry a scale per sub-block (sc: the four float4 that hold the scales of the 16
// rows this lane has results of): the integer sums of the sub-block alone (|64 h + l| <= 32 * 127 * 2^12 < 2^24: exact in
// fp32) times the weights' scale, then times the row's scale of this sub-block into the fp32 result.
template <class W> __device__ __forceinline__ void acc_block_fold(Acc<W> & a, const v16i * s, const typename W::DRec & r, int ib, const float4 * sc) {
    float t[16];
    if constexpr (W::kFoldSub) {
        const float d = W::d_sub(r, ib);
#pragma unroll
        for (int i = 0; i < 16; ++i) t[i] = __fmul_rn(float(s[0][i]), d);
        if constexpr (W::kMin) {   // the second plane is the sum of the row's values
            const float m = -W::dmin_sub(r, ib);
#pragma unroll
            for (int i = 0; i < 16; ++i) t[i] = __fmaf_rn(float(s[1][i]), m, t[i]);
        }
    } else {
        const float d = W::d(r);
#pragma unroll
        for (int i = 0; i < 16; ++i) t[i] = __fmul_rn(float((s[0][i] << 6) + s[1][i]), d);
        if constexpr (W::kMin) {
            const float m = -W::dmin(r);
#pragma unroll
            for (int i = 0; i < 16; ++i) t[i] = __fmaf_rn(float(s[2][i]), m, t[i]);
        }
    }
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        a.sum[4 * c] = __fmaf_rn(t[4 * c], sc[c].x, a.sum[4 * c]);
        a.sum[4 * c + 1] = __fmaf_rn(t[4 * c + 1], sc[c].y, a.sum[4 * c + 1]);
        a.sum[4 * c + 2] = __fmaf_rn(t[4 * c + 2], sc[c].z, a.sum[4 * c + 2]);
        a.sum[4 * c + 3] = __fmaf_rn(t[4 * c + 3], sc[c].w, a.sum[4 * c + 3]);
    }
}
// two consecutive sub-blocks: both sets of products are issued before the first is scaled, so that the matrix pipe works
// through the second while the vector pipe scales the first
template <class W> __device__ __forceinline__ void acc_step2_blocks(Acc<W> & a, v4i x0, v4i x1, const v4i * w0, const v4i * w1, const typename W::DRec & r, int ib0,
                                                                   const float4 * sc0, const float4 * sc1) {
    static_assert(!W::kFp8, "a scale per sub-block: int8 operands only");
    const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    v16i s0[W::kPlanes], s1[W::kPlanes];
#pragma unroll
    for (int p = 0; p < W::kPlanes; ++p) s0[p] = __builtin_amdgcn_mfma_i32_32x32x32_i8(x0, w0[p], zero, 0, 0, 0);
#pragma unroll
    for (int p = 0; p < W::kPlanes; ++p) s1[p] = __builtin_amdgcn_mfma_i32_32x32x32_i8(x1, w1[p], zero, 0, 0, 0);
    // The result is pinned after each scaling: where the loop body is several basic blocks (a format whose decode
    // branches) the compiler otherwise moves the scaling of every sub-block behind the last of them and keeps all their
    // integer sums until then, far more than the registers hold.
    acc_block_fold(a, s0, r, ib0, sc0);
    asm volatile("" : "+v"(a.sum));
    acc_block_fold(a, s1, r, ib0 + 1, sc1);
    asm volatile("" : "+v"(a.sum));
}
// |64 acc_h + acc_l| <= 256 * 127 * 2^12 < 2^28: exact in int32, then one rounding into fp32
template <class W> __device__ __forceinline__ void acc_fold(Acc<W> & a, const typename W::DRec & r) {
    if constexpr (!W::kFp8 && !W::kFoldSub) {
        const float d = W::d(r);
#pragma unroll
        for (int i = 0; i < 16; ++i) a.sum[i] = fold_sb(a.sum[i], a.plane[0][i], a.plane[1][i], d);
        if constexpr (W::kMin) {
            const float m = -W::dmin(r);
#pragma unroll
            for (int i = 0; i < 16; ++i) a.sum[i] = __fmaf_rn(float(a.plane[2][i]), m, a.sum[i]);
        }
    }
}

// dynamic LDS: [2 stages][NB][planes][8 sub-blocks][64 lanes] v4i of decoded weights.
// WAVES waves (8 with two operand slots, 4 with one). Decoding: the 8 * NB (slot, sub-block) pieces of a super-block are
// dealt to the waves in order, 8 NB / WAVES each. Products: a wave takes 8 / WAVES row tiles (tile `wave`, then every
// WAVES-th) against every slot.
// GATEUP: the two slots are the gate and the up bank and SwiGLU joins them; else a plain product (a kernel name of its own
// for each, so that a trace tells them apart)
// BLK: the rows carry a scale per 32-value sub-block (k.xbs): every sub-block's integer sums are scaled on their own
template <int NB, class W, int WAVES, bool GATEUP, bool BLK = false>
__global__ __launch_bounds__(64 * WAVES) void plane_gemm_k(GemmArgs k) {
    constexpr int THREADS = 64 * WAVES, P = W::kPlanes;
    constexpr int TPW = (WAVES == 8 && W::kWideChunks ? 16 : 8) / WAVES;   // row tiles per wave of a shared chunk
    constexpr int PIECES = 8 * NB / WAVES;   // (slot, sub-block) pieces a wave decodes per super-block
    constexpr int SPW = 4 * NB / WAVES;      // operand slots per wave on a lone row tile
    // row tiles per chunk: twice the usual with eight waves where the format's accumulators leave the registers for two row
    // tiles a wave (a chunk's weights are decoded once for twice the rows, and an expert with nine to sixteen row tiles is one
    // item per unit group instead of a full chunk and a lone tile)
    constexpr int CT = WAVES == 8 && W::kWideChunks ? 2 * kChunkTiles : kChunkTiles;
    static_assert((PIECES == 2 || PIECES == 4) && (SPW == 1 || SPW == 2), "wave arrangement");
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    v4i * bs = reinterpret_cast<v4i *>(lds);
    __shared__ __attribute__((aligned(16))) uint8_t s_tab[W::kTabBytes];
    __shared__ uint32_t s_lat[W::kLattice];
    __shared__ int s_asg[(WAVES == 8 && W::kWideChunks ? 16 : 8) * 32];
    __shared__ float s_scale[(WAVES == 8 && W::kWideChunks ? 16 : 8) * 32];
    // the experts' index (chunk and tile prefix sums, counts, offsets), copied once: every item looks its expert up, and a
    // binary search is a chain of dependent reads
    __shared__ int s_cbase[kPlanExperts + 1], s_tbase[kPlanExperts + 1], s_cnt[kPlanExperts + 1], s_off[kPlanExperts + 1];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, n = lane & 31, g = lane >> 5;
    const int mg = wave & 3, nbw = wave >> 2;     // lone row tile: weight tile of the wave within the item, operand slot (SPW == 1)
    const int * plan_chunks = (WAVES == 8 && W::kWideChunks) ? k.plan.chunk_base2 : k.plan.chunk_base;
    const bool cached = k.experts <= kPlanExperts;
    if (cached)
        for (int i = tid; i <= k.experts; i += THREADS) {
            s_cbase[i] = plan_chunks[i];
            s_tbase[i] = k.plan.tile_base[i];
            s_cnt[i] = i < k.experts ? k.counts[i] : 0;
            s_off[i] = k.offsets[i];
        }
    W::tables(s_tab, s_lat, tid, THREADS);
    // Work items are (chunk of row tiles, unit of weight rows). Items that share operand A (one chunk, all units) have
    // indices that agree modulo 8, and the blocks that the round-robin of blocks over the 8 XCDs puts on one XCD take the
    // items of one residue from a counter of their own: one XCD's L2 serves a chunk's rows, and a block that finishes
    // early takes more items. The next ticket is fetched under the current item's work. A block whose own counter has
    // run out goes on with the next XCD's, and so round all eight: the chunks of a residue differ in cost (a lone row tile
    // against eight), so the XCDs' shares differ by a tenth and more, and only the last items of a launch lose their L2.
    // The last block to leave clears the counters for the next launch over these rows.
    __syncthreads();
    const int * cbase = cached ? s_cbase : plan_chunks, * tbase = cached ? s_tbase : k.plan.tile_base;
    const int * cnts = cached ? s_cnt : k.counts, * offs = cached ? s_off : k.offsets;
    const int n_chunks = cbase[k.experts];
    const int groups = k.units / k.unit_group;                  // unit groups per chunk
    const int items_padded = (n_chunks + 7) / 8 * 8 * groups;
    const int NSB = k.b0.cols / 256, rows = k.b0.rows;
    __shared__ int s_ticket;
    int * ctr = k.plan.counters;
    int xcd = int(blockIdx.x) & 7, queues_done = 0;   // the queue this block takes from: its own XCD's first
    int ticket = 0;
    if (tid == 0) ticket = atomicAdd(&ctr[xcd], 1);
    for (;;) {
        __syncthreads();          // the previous item's epilogue has read s_asg / s_scale, the exchange space and s_ticket
        if (tid == 0) s_ticket = ticket;
        __syncthreads();
        const int item = 8 * s_ticket + xcd;
        if (item >= items_padded) {
            if (++queues_done == 8) break;
            xcd = (xcd + 1) & 7;
            if (tid == 0) ticket = atomicAdd(&ctr[xcd], 1);
            continue;
        }
        if (tid == 0) ticket = atomicAdd(&ctr[xcd], 1);
        const int ug = (item >> 3) % groups, chunk = item / (8 * groups) * 8 + (item & 7);
        if (chunk >= n_chunks) continue;
        const int e = owner_of(cbase, k.experts, chunk);
        const int local = chunk - cbase[e], tile_base = tbase[e];
        const bool is_shared = e == k.shared_expert;
        const int u0 = ug * k.unit_group;                                   // the item's first unit
        // gate / up rows of the shared expert beyond its size: no products, zeros stored (the rows are quantised whole later)
        const int live_units = GATEUP && is_shared ? min(max(k.shared_lim / 32 - u0, 0), k.unit_group) : k.unit_group;
        const int sb_full = !GATEUP && is_shared ? k.shared_lim / 256 : NSB;   // super-blocks of a live unit's products
        const int cnt = cnts[e], tiles_e = (cnt + 31) >> 5;
        const int first_tile = local * CT;                                  // of this expert
        const int live_tiles = min(CT, tiles_e - first_tile);               // of this block
        // A chunk of one row tile has nothing for the waves to share: every wave then takes the tile against 32 weight
        // rows of its own (of every slot it has), four units a pass, the chunk's items taking passes in turn.
        const bool lone = live_tiles == 1 && k.units % 4 == 0;
        if (lone && ug >= k.units / 4) continue;
        // the rows' assignments and scales are only read when the results are stored: their loads are issued here and land
        // in LDS after the products, so that nothing waits for them
        constexpr int RPT = (CT * 32 + THREADS - 1) / THREADS;   // rows per thread
        int row_asg[RPT];
        float row_scale[RPT];
#pragma unroll
        for (int q = 0; q < RPT; ++q) {
            const int i = tid + q * THREADS, idx = first_tile * 32 + i;
            row_asg[q] = -1;
            row_scale[q] = 0.f;
            if (i < live_tiles * 32 && idx < cnt) {
                row_asg[q] = k.perm[offs[e] + idx];
                row_scale[q] = k.xs[int64_t(tile_base + first_tile) * 32 + i];
            }
        }
        auto rows_to_lds = [&]() {
#pragma unroll
            for (int q = 0; q < RPT; ++q)
                if (tid + q * THREADS < CT * 32) { s_asg[tid + q * THREADS] = row_asg[q]; s_scale[tid + q * THREADS] = row_scale[q]; }
            __syncthreads();
        };
        if (lone) for (int unit = ug; unit < k.units / 4; unit += groups) {
            // weight tiles of this wave: gate / up: tile 4 unit + mg of bank b; down: tile (4 unit + mg) NB + b; b = the wave's
            // slot, or both slots
            int wt[SPW];
            typename W::Src wsrc[SPW];
            int sbe = 0;
#pragma unroll
            for (int q = 0; q < SPW; ++q) {
                const int b = SPW == 1 ? nbw : q;
                wt[q] = GATEUP ? 4 * unit + mg : (4 * unit + mg) * NB + b;
                wsrc[q] = W::src(b ? k.b1 : k.b0, e, wt[q], n, g);
            }
            {
                const bool wdead = GATEUP && is_shared && wt[0] * 32 >= k.shared_lim;   // gate / up: the slots share the tile number
                sbe = wdead ? 0 : !GATEUP && is_shared ? k.shared_lim / 256 : NSB;
            }
            const int8_t * a_ptr = k.xq + int64_t(tile_base + first_tile) * 32 * k.b0.cols + lane * 16;
            // (row scales per sub-block: the four float4 of the lane's 16 result rows, 8 c + 4 g + 0..3)
            [[maybe_unused]] const float * sc_ptr = BLK ? k.xbs + int64_t(tile_base + first_tile) * (k.b0.cols / 32) * 32 + 4 * g : nullptr;
            // (the weights' codes run a super-block ahead, and so do the row tile's operands where the codes are short; with
            // codes of 12 bytes and more the operands are read at the start of their super-block's work instead: they come
            // from the L2, the SIMD's other wave covers the wait, and a second set of them is 32 registers that those
            // formats spilled)
            constexpr bool kAheadA = sizeof(typename W::Code) <= 8 && !BLK;   // (with a scale per sub-block the second set does not fit beside the sums and scales)
            struct Stage { typename W::Code code[SPW][8]; typename W::Rec rec[SPW]; typename W::DRec drec[SPW]; v4i a[kAheadA ? 8 : 1]; };
            auto fetch1 = [&](int sb, Stage & st) {   // a super-block of the wave's weights and of the row tile
#pragma unroll
                for (int q = 0; q < SPW; ++q) {
                    st.rec[q] = W::rec(wsrc[q], sb);
                    if constexpr (!W::kFp8) st.drec[q] = W::drec(wsrc[q], sb);
                }
#pragma unroll
                for (int ib = 0; ib < 8; ++ib) {
#pragma unroll
                    for (int q = 0; q < SPW; ++q) st.code[q][ib] = W::code(wsrc[q], sb * 8 + ib);
                    if constexpr (kAheadA) st.a[ib] = *reinterpret_cast<const v4i *>(a_ptr + (int64_t(sb) * 8 + ib) * 1024);
                }
            };
            Acc<W> acc[SPW];
#pragma unroll
            for (int q = 0; q < SPW; ++q) acc_clear(acc[q]);
            auto work1 = [&](int sb, Stage & cur, Stage & nxt) {
                v4i a[8];
#pragma unroll
                for (int ib = 0; ib < 8; ++ib) {
                    if constexpr (kAheadA) a[ib] = cur.a[ib];
                    else a[ib] = *reinterpret_cast<const v4i *>(a_ptr + (int64_t(sb) * 8 + ib) * 1024);
                }
                fetch1(min(sb + 1, sbe - 1), nxt);   // past the last one the same again, from the cache: no branch, the same loads in flight on every path
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int ib = 0; ib < 8; ib += 2) {
                    [[maybe_unused]] float4 sc[2][4];
                    if constexpr (BLK) {   // (fenced: started all at the top, the scales of a super-block are more than the registers hold)
                        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                        for (int h = 0; h < 2; ++h)
#pragma unroll
                            for (int c = 0; c < 4; ++c) sc[h][c] = *reinterpret_cast<const float4 *>(sc_ptr + (int64_t(sb) * 8 + ib + h) * 32 + 8 * c);
                    }
#pragma unroll
                    for (int q = 0; q < SPW; ++q) {
                        v4i w0[P], w1[P];
                        W::planes(cur.code[q][ib], cur.rec[q], ib, g, s_tab, s_lat, w0);
                        W::planes(cur.code[q][ib + 1], cur.rec[q], ib + 1, g, s_tab, s_lat, w1);
                        if constexpr (BLK) acc_step2_blocks(acc[q], a[ib], a[ib + 1], w0, w1, cur.drec[q], ib, sc[0], sc[1]);
                        else acc_step2(acc[q], a[ib], a[ib + 1], w0, w1, ib == 0, cur.drec[q], ib);
                    }
                }
                if constexpr (!BLK) {
#pragma unroll
                    for (int q = 0; q < SPW; ++q) acc_fold(acc[q], cur.drec[q]);
                }
            };
            if (sbe > 0) {
                Stage s0, s1;
                fetch1(0, s0);
                for (int sb = 0; sb < sbe; sb += 2) {
                    work1(sb, s0, s1);
                    if (sb + 1 < sbe) work1(sb + 1, s1, s0);
                }
            }
            if constexpr (W::kRowMul) {
#pragma unroll
                for (int q = 0; q < SPW; ++q) {
                    const float rm = W::rowmul((SPW == 1 ? nbw : q) ? k.b1 : k.b0, e, wt[q], n);
#pragma unroll
                    for (int i = 0; i < 16; ++i) acc[q].sum[i] = __fmul_rn(acc[q].sum[i], rm);
                }
            }
            rows_to_lds();
            float * ex = reinterpret_cast<float *>(lds);
            constexpr bool kExchange = SPW == 1 && NB == 2;   // gate and up of a weight tile sit in two waves
            if (GATEUP && kExchange) {   // the up waves hand their sums to the gate waves of the same weight tile
                if (nbw == 1) {
#pragma unroll
                    for (int i = 0; i < 16; ++i) ex[(mg * 16 + i) * 64 + lane] = acc[0].sum[i];
                }
                __syncthreads();
            }
            if (!(GATEUP && kExchange && nbw == 1)) {
                int asg[16];
                float scl[16];
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const int m = 8 * (i >> 2) + 4 * g + (i & 3);   // result register i of lane half g: row m of the tile, weight row n
                    asg[i] = s_asg[m];
                    scl[i] = s_scale[m];
                }
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    if (asg[i] < 0) continue;
                    uint16_t * o = k.out + int64_t(asg[i]) * rows;
                    if (GATEUP) {
                        const float up = kExchange ? ex[(mg * 16 + i) * 64 + lane] : acc[SPW - 1].sum[i];
                        o[wt[0] * 32 + n] = swiglu_half(acc[0].sum[i], up, scl[i], k.glu);
                    } else {
#pragma unroll
                        for (int q = 0; q < SPW; ++q) o[wt[q] * 32 + n] = scaled_half(acc[q].sum[i], scl[i], k.out_bf16);
                    }
                }
            }
        }
        if (lone) continue;
        // Each wave takes TPW row tiles of the chunk (tile `wave`, then every WAVES-th) against the weights of every operand
        // slot: a loaded piece of operand A serves the products with gate and with up (or with both weight tiles of a down
        // unit), and SwiGLU pairs values the same lane holds. The item's units follow each other as one stream of
        // super-blocks: the first weights of unit u + 1 are fetched and decoded under the last products of unit u, so that only
        // the item's first super-block is waited for.
        int my_tiles = 0;
#pragma unroll
        for (int t = 0; t < TPW; ++t) my_tiles += wave + WAVES * t < live_tiles ? 1 : 0;
        const int8_t * a_base = k.xq + int64_t(tile_base + first_tile + wave) * 32 * k.b0.cols + lane * 16;
        const int64_t a_tile = int64_t(WAVES) * 32 * k.b0.cols;
        [[maybe_unused]] const float * sc_base = BLK ? k.xbs + int64_t(tile_base + first_tile + wave) * (k.b0.cols / 32) * 32 + 4 * g : nullptr;
        [[maybe_unused]] const int64_t sc_tile = int64_t(WAVES) * (k.b0.cols / 32) * 32;

        // the weights this wave decodes for everybody: pieces wave * PIECES + q, piece = (slot, sub-block) = (id / 8, id % 8)
        // (gate / up: the unit's 32 rows of the slot's bank; down: row tile NB * unit + slot)
        const int my_slot = wave * PIECES / 8, my_ib0 = wave * PIECES % 8;
        auto weight_tile = [&](int u, int b) { return GATEUP ? u : NB * u + b; };

        // The stream is instantiated per number of live row tiles of the wave (0..TPW), so that its body is one straight
        // line of code the scheduler can interleave. Every instance passes the same barriers.
        auto body = [&](auto mt_tag) {
            constexpr int MT = decltype(mt_tag)::value;
            constexpr int MTA = MT ? MT : 1;
            Acc<W> acc[MTA][NB];
#pragma unroll
            for (int t = 0; t < MTA; ++t)
#pragma unroll
                for (int b = 0; b < NB; ++b) acc_clear(acc[t][b]);
            // the results of unit u (acc) to memory; result register i of lane half g is tile row 8 (i / 4) + 4 g + i % 4, weight
            // row n. The rows' assignments and scales are read first, all at once: a read per element inside the store loop
            // would serialise on LDS latency.
            auto store_unit = [&](int u, bool zero) {
                if constexpr (W::kRowMul) {
#pragma unroll
                    for (int b = 0; b < NB; ++b) {
                        const float rm = W::rowmul(b ? k.b1 : k.b0, e, weight_tile(u, b), n);
#pragma unroll
                        for (int t = 0; t < MT; ++t)
#pragma unroll
                            for (int i = 0; i < 16; ++i) acc[t][b].sum[i] = __fmul_rn(acc[t][b].sum[i], rm);
                    }
                }
#pragma unroll
                for (int t = 0; t < MT; ++t) {
                    int asg[16];
                    float scl[16];
#pragma unroll
                    for (int i = 0; i < 16; ++i) {
                        const int m = (wave + WAVES * t) * 32 + 8 * (i >> 2) + 4 * g + (i & 3);
                        asg[i] = s_asg[m];
                        scl[i] = s_scale[m];
                    }
#pragma unroll
                    for (int i = 0; i < 16; ++i) {
                        if (asg[i] < 0) continue;
                        uint16_t * o = k.out + int64_t(asg[i]) * rows;
                        if (GATEUP) {
                            o[u * 32 + n] = zero ? uint16_t(0) : swiglu_half(acc[t][0].sum[i], acc[t][NB - 1].sum[i], scl[i], k.glu);
                        } else {
#pragma unroll
                            for (int b = 0; b < NB; ++b) o[(NB * u + b) * 32 + n] = zero ? uint16_t(0) : scaled_half(acc[t][b].sum[i], scl[i], k.out_bf16);
                        }
                    }
                }
            };

            // a stream over the units [ub, ub + nu) of the item
            auto run = [&](int ub, int nu) {
            const int total = nu * sb_full, pairs_u = sb_full * 4;

            // Loads run ahead of the products through the item's (unit, super-block) steps: codes and scale records two
            // steps (decoded one step ahead), the fold's scales one step, operand A kSlots - 1 pairs of sub-blocks. Past a
            // unit's last step they go on into the next unit's first ones; past the item's last step they repeat it (from
            // the cache, feeding nothing): selects between two base pointers, no branches around loads.
            typename W::Rec f_rec = {};
            typename W::Code f_code[PIECES] = {};
            typename W::DRec d_rec[NB] = {}, d_rec_next[NB] = {};
            typename W::Src src_cur = W::src(my_slot ? k.b1 : k.b0, e, weight_tile(ub, my_slot), n, g), src_nxt = src_cur;
            typename W::Src dsrc_cur[NB], dsrc_nxt[NB];
#pragma unroll
            for (int b = 0; b < NB; ++b) dsrc_nxt[b] = dsrc_cur[b] = W::src(b ? k.b1 : k.b0, e, weight_tile(ub, b), n, g);
            bool last = nu <= 1;
            // step `ahead` steps after super-block sb of the current unit: in this unit, in the next one, or the item's last
            auto fetch = [&](int sb, int ahead) {
                const int t = sb + ahead;
                const bool here = t < sb_full || last;
                const typename W::Src & src = here ? src_cur : src_nxt;
                const int at = t < sb_full ? t : last ? sb_full - 1 : t - sb_full;
                f_rec = W::rec(src, at);
#pragma unroll
                for (int j = 0; j < PIECES; ++j) f_code[j] = W::code(src, at * 8 + my_ib0 + j);
            };
            auto fetch_d = [&](int sb, int ahead) {
                if constexpr (!W::kFp8) {
                    const int t = sb + ahead;
                    const bool here = t < sb_full || last;
                    const int at = t < sb_full ? t : last ? sb_full - 1 : t - sb_full;
#pragma unroll
                    for (int b = 0; b < NB; ++b) d_rec_next[b] = W::drec(here ? dsrc_cur[b] : dsrc_nxt[b], at);
                }
            };
            auto decode_one = [&](int buf, int j) {
                const int ib = my_ib0 + j;
                v4i w[P];
                W::planes(f_code[j], f_rec, ib, g, s_tab, s_lat, w);
#pragma unroll
                for (int p = 0; p < P; ++p) bs[(((buf * NB + my_slot) * P + p) * 8 + ib) * 64 + lane] = w[p];
            };
            // operand A (the same rows for every unit), two k-steps (sub-blocks) per slot
            constexpr int kSlots = 4;
            v4i a_reg[kSlots][MTA][2];
            auto load_a = [&](int slot, int pair) {   // pair counted from the current unit's first
                const int at = pair < pairs_u ? pair : last ? pairs_u - 1 : pair - pairs_u;
#pragma unroll
                for (int t = 0; t < MT; ++t)
#pragma unroll
                    for (int h = 0; h < 2; ++h) a_reg[slot][t][h] = *reinterpret_cast<const v4i *>(a_base + t * a_tile + (int64_t(at) * 2 + h) * 1024);
            };
            if (total > 0) {
                if (!last) {
                    src_nxt = W::src(my_slot ? k.b1 : k.b0, e, weight_tile(ub + 1, my_slot), n, g);
#pragma unroll
                    for (int b = 0; b < NB; ++b) dsrc_nxt[b] = W::src(b ? k.b1 : k.b0, e, weight_tile(ub + 1, b), n, g);
                }
                fetch(0, 0);
                fetch_d(0, 0);
#pragma unroll
                for (int q = 0; q < kSlots - 1; ++q) load_a(q, q);
#pragma unroll
                for (int j = 0; j < PIECES; ++j) decode_one(0, j);
                fetch(0, 1);
            }
            __syncthreads();
            int parity = 0;   // stage that holds the current unit's first super-block
            for (int uu = 0; uu < (total > 0 ? nu : 0); ++uu) {
                for (int sb = 0; sb < sb_full; ++sb) {
                    const int buf = (parity + sb) & 1;
#pragma unroll
                    for (int b = 0; b < NB; ++b) d_rec[b] = d_rec_next[b];
                    // The decode of the next step's pieces is placed between the groups of products, so that its vector
                    // work runs while the matrix pipe works through the group just issued: in front of the step's last
                    // group where a wave has two pieces, so that the codes (fetched behind the previous step's decode, from
                    // memory) have had a whole step to arrive; the fetch of the step after next follows at once.
                    fetch_d(sb, 1);
#pragma unroll
                    for (int jp = 0; jp < 4; ++jp) {
                        if constexpr (PIECES == 2) {
                            if (jp == 3) { __builtin_amdgcn_sched_barrier(0); decode_one(buf ^ 1, 0); decode_one(buf ^ 1, 1); __builtin_amdgcn_sched_barrier(0); }
                        } else {
                            __builtin_amdgcn_sched_barrier(0); decode_one(buf ^ 1, jp); __builtin_amdgcn_sched_barrier(0);
                        }
                        if (jp == 3) { __builtin_amdgcn_sched_barrier(0); fetch(sb, 2); __builtin_amdgcn_sched_barrier(0); }
                        load_a((jp + kSlots - 1) % kSlots, sb * 4 + jp + kSlots - 1);
                        if constexpr (BLK) {
                            // a group at a time, fenced: its row scales, then each slot's weights and products (started all at
                            // once, the scales and integer sums of a whole step are more than the registers hold)
                            __builtin_amdgcn_sched_barrier(0);
                            float4 sc[MTA][2][4];
#pragma unroll
                            for (int t = 0; t < MT; ++t)
#pragma unroll
                                for (int h = 0; h < 2; ++h)
#pragma unroll
                                    for (int c = 0; c < 4; ++c)
                                        sc[t][h][c] = *reinterpret_cast<const float4 *>(sc_base + t * sc_tile + (int64_t(sb) * 8 + 2 * jp + h) * 32 + 8 * c);
#pragma unroll
                            for (int b = 0; b < NB; ++b) {
                                v4i w0[P], w1[P];
#pragma unroll
                                for (int p = 0; p < P; ++p) {
                                    w0[p] = bs[(((buf * NB + b) * P + p) * 8 + 2 * jp) * 64 + lane];
                                    w1[p] = bs[(((buf * NB + b) * P + p) * 8 + 2 * jp + 1) * 64 + lane];
                                }
#pragma unroll
                                for (int t = 0; t < MT; ++t)
                                    acc_step2_blocks(acc[t][b], a_reg[jp % kSlots][t][0], a_reg[jp % kSlots][t][1], w0, w1, d_rec[b], 2 * jp, sc[t][0], sc[t][1]);
                                __builtin_amdgcn_sched_barrier(0);
                            }
                        } else
#pragma unroll
                        for (int b = 0; b < NB; ++b) {
                            v4i w0[P], w1[P];
#pragma unroll
                            for (int p = 0; p < P; ++p) {
                                w0[p] = bs[(((buf * NB + b) * P + p) * 8 + 2 * jp) * 64 + lane];
                                w1[p] = bs[(((buf * NB + b) * P + p) * 8 + 2 * jp + 1) * 64 + lane];
                            }
#pragma unroll
                            for (int t = 0; t < MT; ++t) acc_step2(acc[t][b], a_reg[jp % kSlots][t][0], a_reg[jp % kSlots][t][1], w0, w1, jp == 0, d_rec[b], 2 * jp);
                        }
                    }
                    if constexpr (!BLK) {
#pragma unroll
                        for (int b = 0; b < NB; ++b)
#pragma unroll
                            for (int t = 0; t < MT; ++t) acc_fold(acc[t][b], d_rec[b]);
                    }
                    __syncthreads();
                }
                if (uu == 0) rows_to_lds();   // the rows' assignments and scales: long arrived
                store_unit(ub + uu, false);
#pragma unroll
                for (int t = 0; t < MTA; ++t)
#pragma unroll
                    for (int b = 0; b < NB; ++b) acc_clear(acc[t][b]);
                // on to the next unit: its first super-block sits in the stage already, its first pairs of operand A in registers
                parity = (parity + sb_full) & 1;
                src_cur = src_nxt;
#pragma unroll
                for (int b = 0; b < NB; ++b) dsrc_cur[b] = dsrc_nxt[b];
                last = uu + 2 >= nu;
                if (!last) {
                    src_nxt = W::src(my_slot ? k.b1 : k.b0, e, weight_tile(ub + uu + 2, my_slot), n, g);
#pragma unroll
                    for (int b = 0; b < NB; ++b) dsrc_nxt[b] = W::src(b ? k.b1 : k.b0, e, weight_tile(ub + uu + 2, b), n, g);
                }
            }
            };
            // (units of a single super-block cannot look two steps ahead into one next unit: they run one by one)
            if (sb_full >= 2) run(u0, live_units);
            else for (int i = 0; i < live_units; ++i) run(u0 + i, 1);
            if (live_units < k.unit_group) {   // units past the shared expert's size: zeros
                if (live_units * sb_full == 0) rows_to_lds();
                for (int u = u0 + live_units; u < u0 + k.unit_group; ++u) store_unit(u, true);
            }
        };
        if constexpr (TPW == 1) {
            if (my_tiles) body(std::integral_constant<int, 1>{}); else body(std::integral_constant<int, 0>{});
        } else {
            static_assert(TPW == 2, "row tiles per wave");
            switch (my_tiles) {
                case 0: body(std::integral_constant<int, 0>{}); break;
                case 1: body(std::integral_constant<int, 1>{}); break;
                default: body(std::integral_constant<int, 2>{}); break;
            }
        }
    }   // items
    if (tid == 0) {
        __threadfence();
        if (atomicAdd(&ctr[8], 1) == int(gridDim.x) - 1)
            for (int i = 0; i < kPlanCounters; ++i) atomicExch(&ctr[i], 0);
    }
}

// Two operand slots run on eight waves (a row tile each). The four-wave arrangement of the same kernel (two row tiles a wave,
// half the LDS reads per product, twice the registers) measured 15 to 20 % slower on every format: one wave per SIMD leaves
// nothing to issue while that wave waits.
template <class W, bool BLK = false> void plane_gemm_launch(int nb, bool gateup, const GemmArgs & k, unsigned blocks, hipStream_t s) {
    const size_t lds = size_t(2) * nb * W::kPlanes * 8 * 64 * sizeof(v4i);
    constexpr size_t kLdsMost = size_t(2) * 2 * 3 * 8 * 64 * sizeof(v4i);
    auto launch = [&](auto kernel, unsigned threads) {
        if (lds > 65536 - 24576) allow_dynamic_lds(reinterpret_cast<const void *>(kernel), kLdsMost);
        kernel<<<blocks, threads, lds, s>>>(k);
    };
    if (gateup) launch(&plane_gemm_k<2, W, 8, true, BLK>, 512);
    else if (nb == 2) launch(&plane_gemm_k<2, W, 8, false, BLK>, 512);
    else launch(&plane_gemm_k<1, W, 4, false, BLK>, 256);
}

}  // namespace
}  // namespace tqmoe

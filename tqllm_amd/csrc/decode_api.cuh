// Types shared by the decode entry points (decode.hip) and the per-format kernel translation units.
#pragma once
#include "common.cuh"

namespace tqmoe {

struct BankView { const uint8_t * codes; const uint8_t * aux; int64_t rows_total; int rows, cols; };
inline BankView view(const tqmoe_bank & b) {
    return BankView{static_cast<const uint8_t *>(b.codes), static_cast<const uint8_t *>(b.aux), int64_t(b.experts) * b.rows, b.rows, b.cols};
}

// lanes per row (8, 16, 32 or 64) and sub-blocks per lane (1..4) for S sub-blocks per row; m == 0: not supported
struct Split { int lpr, m; };
inline Split split_for(int S, int64_t assignments = 1 << 30) {
    if (S % 64 == 0) return Split{64, S / 64 <= 4 ? S / 64 : 0};
    // 17 to 31 sub-blocks, a few assignments: a lane per sub-block with the last lanes of each 32 idle, rather than three
    // sub-blocks per lane on 8 lanes. Three times the activation blocks in registers (190 and more) leave a SIMD two waves
    // instead of five, and a short batch is a chain of trips to memory that only more waves shorten (one token: 15 % of the
    // step); a long batch is bound by the vector work, and the idle lanes then cost more (64 tokens: +8 %).
    if (S > 16 && S < 32 && assignments <= 48) return Split{32, 1};
    for (int lpr = 32; lpr >= 8; lpr >>= 1)
        if (S % lpr == 0 && S / lpr <= 4 && (S / lpr == 1 || S / lpr == 3)) return Split{lpr, S / lpr};
    return Split{64, (S + 63) / 64 <= 4 ? (S + 63) / 64 : 0};  // ragged: lanes past the row's last sub-block idle
}

struct MatvecArgs {
    BankView b0, b1;
    const uint8_t * image;
    void * y0, * y1;
    uint32_t ytype;
    const int * ids;
    int A, xdiv, mode, slots, topk, shared_cols;
};
struct GateupArgs {
    BankView bg, bu;
    const uint8_t * ximage;
    uint8_t * aimage;
    const int * ids;
    int A, slots, topk, shared_ff, mode;
    Glu glu;                  // the optional clamp of the SwiGLU inputs
};

// arguments of the grouped fp16 products (prefill_f16_kernels.cuh)
struct F16Args {
    BankView b0, b1;
    const void * x;           // input rows of xtype, cols = bank cols
    uint32_t xtype;
    const int * counts;       // [experts]
    const int * offsets;      // [experts + 1]
    const int * perm;         // assignment indices grouped by expert
    int experts;
    int xdiv;                 // input row of assignment a = a / xdiv
    void * out;               // [assignments][rows]
    uint32_t out_type;        // TQMOE_F16, TQMOE_BF16 or TQMOE_F32
    int gateup;
    int shared_expert;        // the expert whose rows (gate / up) or columns (down) stop at shared_lim, or -1
    int shared_lim;
    Glu glu;                  // gateup: the optional clamp of the SwiGLU inputs
};
// the grouped fp16 product of one bank format; wide: 128 input rows per block (grid.y counts such units), else 64
template <uint32_t FMT> struct F16Launch {
    static void run(const F16Args & k, bool two_banks, bool wide, dim3 grid, hipStream_t s);
};

// launch tables, one explicit instantiation per bank format (decode_<format>.hip)
template <uint32_t FMT> struct DecodeLaunch {
    static void matvec(Split sp, int nb, const MatvecArgs & k, hipStream_t s);
    static void gateup(Split sp, const GateupArgs & k, hipStream_t s);
};
template <> void DecodeLaunch<TQMOE_IQ4_XS>::matvec(Split sp, int nb, const MatvecArgs & k, hipStream_t s);   // its own kernels (decode_iq4xs.hip)
template <> void DecodeLaunch<TQMOE_IQ4_XS>::gateup(Split sp, const GateupArgs & k, hipStream_t s);
extern template struct DecodeLaunch<TQMOE_Q4_K>;
extern template struct DecodeLaunch<TQMOE_IQ3_S>;
extern template struct DecodeLaunch<TQMOE_NVFP4G>;
extern template struct DecodeLaunch<TQMOE_IQ4_NL>;
extern template struct DecodeLaunch<TQMOE_Q8_0>;
extern template struct DecodeLaunch<TQMOE_Q5_K>;
extern template struct DecodeLaunch<TQMOE_Q6_K>;
extern template struct DecodeLaunch<TQMOE_IQ3_XXS>;
extern template struct DecodeLaunch<TQMOE_IQ2_S>;
extern template struct DecodeLaunch<TQMOE_Q2_K>;
extern template struct DecodeLaunch<TQMOE_IQ1_S>;
extern template struct DecodeLaunch<TQMOE_Q4_0>;
extern template struct DecodeLaunch<TQMOE_Q3_K>;
extern template struct DecodeLaunch<TQMOE_IQ2_XXS>;
extern template struct DecodeLaunch<TQMOE_IQ2_XS>;
extern template struct F16Launch<TQMOE_IQ4_XS>;
extern template struct F16Launch<TQMOE_Q4_K>;
extern template struct F16Launch<TQMOE_IQ3_S>;
extern template struct F16Launch<TQMOE_NVFP4G>;
extern template struct F16Launch<TQMOE_IQ4_NL>;
extern template struct F16Launch<TQMOE_Q8_0>;
extern template struct F16Launch<TQMOE_Q5_K>;
extern template struct F16Launch<TQMOE_Q6_K>;
extern template struct F16Launch<TQMOE_IQ3_XXS>;
extern template struct F16Launch<TQMOE_IQ2_S>;
extern template struct F16Launch<TQMOE_Q2_K>;
extern template struct F16Launch<TQMOE_IQ1_S>;
extern template struct F16Launch<TQMOE_Q4_0>;
extern template struct F16Launch<TQMOE_Q3_K>;
extern template struct F16Launch<TQMOE_IQ2_XXS>;
extern template struct F16Launch<TQMOE_IQ2_XS>;

}  // namespace tqmoe

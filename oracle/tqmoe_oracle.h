/* CPU oracle for the mixture-of-experts layer: TEST INFRASTRUCTURE ONLY.
 *
 * A plain, single-purpose restatement of the reference's host algorithms for this path. Only tests, the smoke check
 * and the CPU-baseline leg of the benchmark may link or load it; the product library never does.
 *
 * What each function follows in the reference (paths relative to the reference tree):
 *   tqo_half_to_float / tqo_float_to_half  src/formats/weight/dequant.cpp:12-54
 *   tqo_e4m3_to_float                      src/formats/weight/dequant.cpp:387-391
 *   tqo_dequantize  Q4_K                   src/formats/weight/dequant.cpp:56-64, 80-99
 *                   IQ3_S                  src/formats/weight/dequant.cpp:133-150
 *                   IQ4_XS                 src/formats/weight/dequant.cpp:176-192
 *                   IQ4_NL                 src/formats/weight/dequant.cpp:351-360
 *                   Q8_0                   src/formats/weight/dequant.cpp:555-562
 *                   Q5_K                   src/formats/weight/dequant.cpp:102-116
 *                   IQ3_XXS                src/formats/weight/dequant.cpp:157-174 (no encoder here: tests use random blocks)
 *                   IQ2_S                  src/formats/weight/dequant.cpp:271-287 (likewise)
 *                   IQ2_XXS, IQ2_XS        src/formats/weight/dequant.cpp:233-249, 252-268 (likewise)
 *                   Q3_K                   src/formats/weight/dequant.cpp:66-76, 118-131 (likewise)
 *                   Q4_0                   src/formats/weight/dequant.cpp:480-491 (likewise)
 *                   Q2_K                   src/formats/weight/dequant.cpp:289-310 (likewise)
 *                   IQ1_S                  src/formats/weight/dequant.cpp:311-326 (likewise)
 *                   Q6_K                   src/formats/weight/dequant.cpp:194-208
 *                   NVFP4G                 src/formats/weight/dequant.cpp:397-409
 *   tqo_route                              src/experts/moe.cpp:22-113 (softmax / sigmoid / softmax-of-selected /
 *                                          sqrt-softplus gating, selection bias, stable top-k, unbiased weights,
 *                                          clamp 6.103515625e-5, scale)
 *   tqo_shared_weight                      src/experts/moe.cu:92 (sigmoid of logits column E)
 *   tqo_dispatch                           src/models/qwen/qwen4exp/prefill_plan.hpp:63-74 (ascending assignment
 *                                          order inside each expert), counts as src/experts/moe.cu:168-176
 *   tqo_add_rmsnorm                        src/formats/weight/quant_tq3.inc:293-313 (add, sums of squares) and
 *                                          src/formats/weight/quant.cu:647-661 (norm), as called by
 *                                          src/models/qwen/qwen35/qwen35_forward.cpp:1114-1115
 *   tqo_expert_ffn                         src/experts/moe.cpp:115-155
 *   tqo_combine                            src/experts/moe.cpp:157-163 and src/experts/moe.cu:224-234 (shared row)
 *   tqo_router_logits                      src/experts/moe.cu:17-33 (row E = shared gate), bf16 variant
 *                                          src/models/qwen/qwen4exp/qwen4exp.cu:1629-1659
 *   tqo_layer_forward                      tests/glm_expert_bank.cu:166-184 (dequantise, route, FFN per selected
 *                                          expert, combine)
 *   tqo_quant_act_row_i8                   src/formats/weight/quant_u4h.inc:790-820 (per-token mode: scale m/127)
 *   tqo_quant_act_blocks_i8                src/formats/weight/quant_u4h.inc:790-822 (per-32-block mode: a scale and two
 *                                          sums of 16 per block)
 *   tqo_quant_act_row_e4m3                 src/core/fp8_gemm.cuh:19-20 (per-row scale amax/448)
 *
 * Pinned by: tests/golden/kquant_golden.bin (gguf-py values, bit for bit) for Q4_K / IQ3_S / IQ4_XS / IQ4_NL; the
 * 65,536 halves against hardware conversion; the 256 E4M3 codes against the closed form; NVFP4G against the closed
 * form value = e2m1 * e4m3(scale) * global; routing against an independent max-scan selection, scipy softmax and
 * the closed forms of the reference's tests/moe.cpp; dispatch against a brute-force stable sort; FFN / combine /
 * layer against float64 numpy on the decoded weights; the residual add and norm against float64 numpy and closed
 * forms (constant rows, zero rows, the eps limit); and, where it builds, against the reference's own objects in
 * oracle/_ref.
 *
 * PARITY UNPINNED: tqo_quantize (all formats). The reference holds no quantiser (it calls an external libggml that
 * is not in its tree); the encoders here are this build's own and are checked only through round trip and block
 * validity. Layer parity is defined on decoded values, so the encoder changes the weight distribution, not the
 * pass criterion.
 */
#ifndef TQMOE_ORACLE_H
#define TQMOE_ORACLE_H
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

/* GGUF tensor type ids (src/core/gguf.hpp) */
enum { TQO_F32 = 0, TQO_F16 = 1, TQO_Q4_0 = 2, TQO_Q8_0 = 8, TQO_Q2_K = 10, TQO_Q3_K = 11, TQO_Q4_K = 12, TQO_Q5_K = 13, TQO_Q6_K = 14, TQO_IQ2_XXS = 16, TQO_IQ2_XS = 17, TQO_IQ3_XXS = 18, TQO_IQ1_S = 19, TQO_IQ2_S = 22, TQO_IQ4_NL = 20, TQO_IQ3_S = 21, TQO_IQ4_XS = 23, TQO_BF16 = 30,
       TQO_NVFP4G = 323 };
/* gating (src/experts/moe.hpp:20-26) */
enum { TQO_GATE_SOFTMAX = 1, TQO_GATE_SIGMOID = 2, TQO_GATE_SOFTMAX_WEIGHT = 3, TQO_GATE_SQRT_SOFTPLUS = 4 };

float    tqo_half_to_float(uint16_t h);
uint16_t tqo_float_to_half(float f);
float    tqo_bf16_to_float(uint16_t h);
uint16_t tqo_float_to_bf16(float f);          /* round to nearest even */
float    tqo_e4m3_to_float(uint8_t b);
uint8_t  tqo_float_to_e4m3(float f);          /* round to nearest even, saturating at +-448 */

/* block layout: weights per block and bytes per block; returns 0 when the type is not one of the five */
int tqo_block_layout(uint32_t type, int * elems, int * bytes);
/* n weights (a multiple of the block size) from GGUF blocks to fp32; returns 0 on success */
int tqo_dequantize(uint32_t type, const void * src, float * dst, int64_t n);
/* n fp32 weights to GGUF blocks (this build's own encoders: parity unpinned); for NVFP4G `row` = weights per
 * matrix row (one global scale per row). Returns 0 on success. */
int tqo_quantize(uint32_t type, const float * src, void * dst, int64_t n, int64_t row);

/* routing of one token: logits[E] (+ optional selection bias[E]) -> ids[k] (descending selection value, ties to
 * the lower index) and weights[k] */
int tqo_route(int gating, int n_expert, int k, int norm_weights, float weight_scale, const float * logits,
              const float * bias, int32_t * ids, float * weights);
/* 1 when, among the k + 1 largest softmax probabilities as tqo_route computes them (ties to the lower index), two
 * neighbours have the same nonzero fp32 probability although their logits differ, or one of them is a subnormal number:
 * the tokens on which a selection by logit (what a kernel with another exp() can reproduce exactly) and the reference's
 * selection by rounded probability may differ. Equal logits, and probabilities that underflowed to zero, are ordered by
 * index on both sides and are no collision. */
int tqo_route_softmax_collision(int n_expert, int k, const float * logits);
float tqo_shared_weight(float logit);

/* stable dispatch: counts[E], offsets[E + 1] (exclusive scan), perm[A] = assignment indices grouped by expert in
 * ascending order inside each expert; ids < 0 are skipped (offsets[E] = number kept) */
int tqo_dispatch(const int32_t * ids, int A, int E, int32_t * counts, int32_t * offsets, int32_t * perm);

void tqo_expert_ffn(const float * x, int hidden, const float * w_gate, const float * w_up, const float * w_down,
                    int ff, float swiglu_clamp, int clamp_gate, float * out);
/* out[hidden] += sum_s weights[s] * expert_outs[s][hidden] */
void tqo_combine(const int k, const float * weights, const float * expert_outs, int hidden, float * out);

/* logits[n][E + 1] = W x, row E from `shared_gate` (may be null: column E = 0). wtype / xtype: TQO_F32, TQO_BF16 or
 * TQO_F16 storage; products and sums in fp32, j ascending. */
int tqo_router_logits(const void * w, uint32_t wtype, const void * shared_gate, const void * x, uint32_t xtype,
                      int hidden, int E, int n, float * logits);

/* Declared activation quantisers of the lossy operand paths. */
void tqo_quant_act_row_i8(const float * x, int cols, int8_t * q, float * scale);     /* scale = amax/127 */
void tqo_quant_act_row_e4m3(const float * x, int cols, uint8_t * q, float * scale);  /* scale = amax/448 */
/* a scale per 32 values (scales[cols / 32]) and the sums of q over each 16 (qsum[cols / 32][2], may be null); cols a multiple of 32 */
void tqo_quant_act_blocks_i8(const float * x, int cols, int8_t * q, float * scales, int16_t * qsum);
/* NVFP4G blocks -> fp32 with e2m1 * (E4M3 scale) / 8 rounded to E4M3 before 8 * the row's global multiplies it: the
 * weights of an fp8 matrix product that keeps the global outside the operand (the 8 keeps 6 * 448 inside E4M3). n a
 * multiple of 128. */
int  tqo_dequantize_nvfp4_widened(const void * src, float * dst, int64_t n);

/* Residual add and RMS norm in front of the layer, the reference's add_sumsq + norm_h with their summation order
 * (per 256 values: xor butterflies over 32, then the eight sums in order; the blocks' sums strided over 32 lanes and
 * a butterfly): rows (bf16 bits, [n][hidden]) += residual in place (skipped when null), normed_bf16 = bf16((row * inv) *
 * weight) with inv = 1 / sqrt(sum / hidden + eps) (the reference's device rsqrtf is approximate; this one is exact).
 * hidden must be a multiple of 256. */
int tqo_add_rmsnorm(uint16_t * rows, const uint16_t * residual, const float * weight, float eps, int hidden, int n,
                    uint16_t * normed_bf16);

/* Whole layer on the host.
 *   x fp32 [n][H] (already rounded to the activation type by the caller), logits [n][E + 1] given (so that the
 *   routing of a device run can be replayed on the device's own logits), banks = GGUF blocks [E (+1)][rows][cols]
 *   for gate, up ([F][H]) and down ([H][F]); shared expert = expert index E of the same banks when has_shared,
 *   its FFN size shared_ff <= F (the first shared_ff rows / columns), weighted by sigmoid(logits[.][E]).
 *   act_mode: 0 = fp32 activations (oracle A); 1 = the inputs of both products (the token row, the act row) passed
 *   through tqo_quant_act_row_i8 (oracle B of an int8 path that keeps fp32 intermediate rows); 5 = mode 1 with
 *   silu(gate) * up and the down product each rounded to fp16 (oracle B of the grouped int8 products, which store
 *   fp16 rows); 6 = mode 5 with a scale per 32 values in place of one per row (tqo_quant_act_blocks_i8: the reference's
 *   per-32-block mode of the same products); 2 = NVFP4G banks on fp8 operands (oracle B of the grouped fp8 products): both product inputs passed
 *   through tqo_quant_act_row_e4m3, the weights through tqo_dequantize_nvfp4_widened, fp16 roundings as in mode 5.
 *   out fp32 [n][H]; ids_out [n][k], weights_out [n][k] may be null. threads: worker threads over tokens.
 *   gating (0 = softmax), raw_weights (nonzero: unnormalised), weight_scale (0 = none) and bias (or null) are
 *   tqo_route's arguments; all zero is softmax routing with normalised weights.
 */
typedef struct tqo_layer {
    int hidden, ff, n_expert, k, has_shared, shared_ff;
    uint32_t wtype;
    const void * gate, * up, * down;
    int act_mode;
    int threads;
    int gating, raw_weights;
    float weight_scale;
    const float * bias;
    uint32_t wtype_down;   /* format of the down bank when it differs from gate / up (0: the same) */
    float swiglu_clamp;    /* MoeConfig::swiglu_clamp of every expert FFN (src/experts/moe.cpp:128-143); <= 1e-6: none */
    int clamp_gate;        /* its clamp_gate switch */
    float * act_out;       /* optional (act modes other than 0): [n * slots][ff] the rows silu(gate) * up as the down product's quantiser
                              receives them (after the fp16 rounding of the modes that have one), row t * slots + s, slots = k + has_shared;
                              a shared row has shared_ff values */
} tqo_layer;
int tqo_layer_forward(const tqo_layer * L, const float * x, const float * logits, int n, float * out,
                      int32_t * ids_out, float * weights_out);

/* CPU baseline: the scheme of the reference's tests/bench_cpu_expert_mt.cpp on this build's bank formats (IQ4_XS,
 * IQ4_NL, Q4_K, IQ3_S, NVFP4G).
 * tqo_cpu_expert_bench: table 1 (:69-116). `threads` workers pull experts from an atomic counter; each expert = gate,
 * up, down matvec of one token with per-32-block int8 activations and AVX2 integer dots (int8_act = 1) or fp32
 * activations (0). Returns seconds per pass over n_expert experts, averaged over `reps` passes after one warm pass.
 * tqo_cpu_expert_latency: table 2 (:130-199). One expert (index 0 of the banks), its rows split over `threads`
 * persistent workers woken by a generation counter, int8 activations; seconds per expert.
 * tqo_cpu_matvec: one matvec y[rows] = W x with the kernels the two benches run. mode 0 fp32, 1 int8 activations
 * with AVX2 integer dots, 2 int8 activations with scalar integer dots. */
double tqo_cpu_expert_bench(uint32_t wtype, const void * gate, const void * up, const void * down, int hidden, int ff,
                            int n_expert, int threads, int int8_act, int reps, float * checksum);
double tqo_cpu_expert_latency(uint32_t wtype, const void * gate, const void * up, const void * down, int hidden, int ff,
                              int threads, int reps, float * checksum);
int tqo_cpu_matvec(uint32_t wtype, const void * W, int rows, int cols, const float * x, int mode, float * y);
int tqo_hardware_threads(void);

#ifdef __cplusplus
}
#endif
#endif

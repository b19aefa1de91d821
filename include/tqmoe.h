/* tqmoe: the mixture-of-experts layer of tqLLM for one AMD Instinct MI355X (gfx950), as a C ABI.
 *
 * The library is what the reference's `src/experts` free functions (namespace tqllm_cuda, moe_kernels.cuh) and the
 * expert entry points of `tqllm::WeightFormat` (src/formats/weight/weight_format.hpp) are to its CUDA engine, with
 * the conventions of the reference's only C ABI (include/tqllm/plugin.h, ABI 2):
 *   - every pointer named `*_dev` or documented "device" is HIP device memory owned by the caller; streams travel as
 *     `void *` (a hipStream_t, NULL = the default stream), so this header needs no GPU include;
 *   - every call only enqueues work on the given stream: no host synchronisation, no allocation, no state kept between
 *     calls (the one-time constant tables live in the library's own device image);
 *   - every call returns 0 on success; on failure a negative TQMOE_E_* code, with the reason in `err` when given
 *     (`err` may be NULL; set err->struct_size = sizeof(tqmoe_error) before the call);
 *   - assignments whose expert id is negative are skipped and their output rows left untouched
 *     (src/formats/weight/quant_u4h.inc:443-447).
 * There is no CPU fallback: without a usable HIP device every compute entry point fails with TQMOE_E_DEVICE.
 */
#ifndef TQMOE_H
#define TQMOE_H
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

#define TQMOE_ABI_VERSION 1u

/* error record, shaped as plugin.h:9 `tq_error` */
typedef struct tqmoe_error { uint32_t struct_size; int32_t code; char message[256]; } tqmoe_error;
enum { TQMOE_OK = 0, TQMOE_E_ARG = -1, TQMOE_E_UNSUPPORTED = -2, TQMOE_E_DEVICE = -3, TQMOE_E_WORKSPACE = -4 };

/* element types (GGUF type ids, src/core/gguf.hpp) */
enum { TQMOE_F32 = 0, TQMOE_F16 = 1, TQMOE_BF16 = 30 };
/* bank formats (GGUF type ids) */
enum { TQMOE_Q4_0 = 2, TQMOE_Q8_0 = 8, TQMOE_Q2_K = 10, TQMOE_Q3_K = 11, TQMOE_Q4_K = 12, TQMOE_Q5_K = 13, TQMOE_Q6_K = 14, TQMOE_IQ2_XXS = 16, TQMOE_IQ2_XS = 17,
       TQMOE_IQ3_XXS = 18, TQMOE_IQ1_S = 19, TQMOE_IQ4_NL = 20, TQMOE_IQ3_S = 21, TQMOE_IQ2_S = 22, TQMOE_IQ4_XS = 23, TQMOE_NVFP4G = 323 };

uint32_t tqmoe_abi_version(void);

/* ------------------------------------------------------------------------------------------------ routing
 * Router logits: logits[t][r] = sum_j W[r][j] * x[t][j] for r < experts, logits[t][experts] = shared_gate . x[t]
 * (0 when shared_gate is NULL); row stride experts + 1; products and sums in fp32.
 * Replaces tqllm_cuda::moe_router / moe_router_f32 (src/experts/moe_kernels.cuh:7-10, moe.cu:17-33, 237-247) and
 * the bf16 segmented GEMV fn_gemv_bf16_segments (src/models/qwen/qwen4exp/qwen4exp.cu:1629-1659).
 * router: device [experts][hidden] of wtype (F32 or BF16); shared_gate: device [hidden] of wtype or NULL;
 * x: device [n][hidden] of xtype (F32, F16 or BF16); logits: device [n][experts + 1] fp32. */
int32_t tqmoe_router(const void * router, uint32_t wtype, const void * shared_gate, const void * x, uint32_t xtype,
                     float * logits, int32_t hidden, int32_t experts, int32_t n, void * stream, tqmoe_error * err);

/* Softmax over the first `experts` columns, the `topk` largest probabilities (descending, ties to the lower index),
 * weights = probability / max(sum of the selected, 6.103515625e-5) * (scale == 0 ? 1 : scale), and
 * shared_weights[t] = sigmoid(logits[t][experts]) (shared_weights may be NULL).
 * Replaces tqllm_cuda::moe_topk (moe_kernels.cuh:19-20, moe.cu:35-166, 248-260); host meaning: moe_route
 * (src/experts/moe.cpp:22-113) with Softmax gating, norm_weights, weight_scale = scale. experts <= 4096. */
int32_t tqmoe_topk(const float * logits, int32_t * ids, float * weights, float * shared_weights, int32_t experts,
                   int32_t topk, int32_t n, float scale, void * stream, tqmoe_error * err);

/* tqmoe_topk on two routings of the same shape in one launch (this layer's and a prediction of the next layer's): the
 * results of the two calls it stands for, bit for bit. Replaces tqllm_cuda::moe_topk2 (moe_kernels.cuh:24-25,
 * moe.cu:261-263; called from src/models/qwen/qwen4exp/fn_layer_forward.cpp:331). experts <= 1024, as there. */
int32_t tqmoe_topk2(const float * logits, int32_t * ids, float * weights, float * shared_weights, const float * logits2,
                    int32_t * ids2, float * weights2, float * shared_weights2, int32_t experts, int32_t topk, int32_t n,
                    float scale, void * stream, tqmoe_error * err);

/* The reference's other routing modes, moe_route (src/experts/moe.cpp:22-113) in full:
 *   gating        TQMOE_GATE_SOFTMAX         p = softmax(logits)
 *                 TQMOE_GATE_SIGMOID         p = 1 / (1 + exp(-logit))
 *                 TQMOE_GATE_SOFTMAX_WEIGHT  p = logit; the weights are a softmax over the selected logits only
 *                 TQMOE_GATE_SQRT_SOFTPLUS   p = sqrt(log(1 + exp(logit)))
 *   probs_bias    device [experts] fp32 or NULL: added to p for the choice only (descending p + bias, ties to the lower
 *                 index); the weights come from the unbiased p
 *   norm_weights  nonzero: weights divided by max(their sum, 6.103515625e-5); then * (scale == 0 ? 1 : scale)
 * The values are MoeGating's (src/experts/moe.hpp:20-26). shared_weights as in tqmoe_topk. experts <= 4096. */
enum { TQMOE_GATE_SOFTMAX = 1, TQMOE_GATE_SIGMOID = 2, TQMOE_GATE_SOFTMAX_WEIGHT = 3, TQMOE_GATE_SQRT_SOFTPLUS = 4 };
int32_t tqmoe_topk_gated(const float * logits, const float * probs_bias, int32_t gating, int32_t norm_weights,
                         int32_t * ids, float * weights, float * shared_weights, int32_t experts, int32_t topk,
                         int32_t n, float scale, void * stream, tqmoe_error * err);

/* Token-to-expert dispatch of the A = n * topk assignments a = t * topk + s:
 *   counts[e]   assignments of expert e (ids < 0 skipped),
 *   offsets[e]  exclusive scan of counts, offsets[experts] = number kept,
 *   perm[i]     assignment indices grouped by expert, ascending inside each expert (a stable counting sort),
 *   groups      optional (NULL to skip) [experts][capacity] view of the same lists, as the reference's kernels read
 *               them; capacity >= the largest count, else TQMOE_E_ARG is NOT detectable on the host and the lists
 *               are truncated at capacity (counts stay exact).
 * Replaces tqllm_cuda::moe_group (moe_kernels.cuh:29, moe.cu:168-176, 268-273; order there is atomic) and the host
 * fill_pass_lists (src/models/qwen/qwen4exp/prefill_plan.hpp:63-74; ascending order). The result is deterministic.
 * workspace: device scratch of tqmoe_dispatch_workspace_bytes(). */
size_t  tqmoe_dispatch_workspace_bytes(int32_t experts, int32_t n, int32_t topk);
int32_t tqmoe_dispatch(const int32_t * ids, int32_t * counts, int32_t * offsets, int32_t * perm, int32_t * groups,
                       int32_t capacity, int32_t experts, int32_t n, int32_t topk, void * workspace,
                       size_t workspace_bytes, void * stream, tqmoe_error * err);

/* tqmoe_dispatch for callers that cannot allocate or carry a workspace (code under HIP graph capture, tight serving
 * loops, harnesses that forbid allocation). It has no counterpart in the reference. Same lists, same kernels; the
 * per-chunk counts live in a 4 MiB array inside the library's device image (one copy per GPU, held until the process
 * ends), whose address is looked up on the first call on a device. Limit: ceil(n * topk / 1024) * experts <= 1,048,576
 * (for 512 experts about two million assignments), beyond it TQMOE_E_WORKSPACE. Calls on one GPU share that array:
 * two calls that overlap in time on the same GPU (different streams) race; calls on one stream are ordered. Nothing
 * in the array needs clearing between calls (every entry a call reads, it has written first).
 * offsets and perm may be NULL when groups is given: counts + groups alone are what tqllm_cuda::moe_group
 * (moe_kernels.cuh:29) produces, and with capacity = n this call is that function with ascending lists.
 * The array's address is looked up on the first call on a device (a module load may happen then): a caller that will
 * capture the call into a HIP graph calls tqmoe_static_scratch_init() once per device beforehand. */
int32_t tqmoe_dispatch_static(const int32_t * ids, int32_t * counts, int32_t * offsets, int32_t * perm, int32_t * groups,
                              int32_t capacity, int32_t experts, int32_t n, int32_t topk, void * stream, tqmoe_error * err);
int32_t tqmoe_static_scratch_init(tqmoe_error * err);

/* counts[ids[i]] += 1 for i < count, 64-bit counters that run on over many calls (ids < 0 skipped): the routing histogram
 * tqllm_cuda::moe_count (moe_kernels.cuh, moe.cu:183-186). */
int32_t tqmoe_count(const int32_t * ids, uint64_t * counts, int32_t count, void * stream, tqmoe_error * err);

/* Slot and de-duplication maps of one routed decode call, tqllm_cuda::moe_dedup_maps (moe_kernels.cuh:34-39, moe.cu:453-493)
 * with the map layout of src/formats/weight/quant_kernels.cuh:26-27 (kDedupCols = 8, kDedupStride = 18):
 *   slots[a] = slot_of[ids[a]] (-1 for ids[a] < 0), a < count <= 1024; slots may be NULL;
 *   gu / dn: `groups` entries of 18 ints each (groups >= count; either may be NULL). The assignments of a slot, in ascending a,
 *   are cut into runs of up to 8; every run is one entry {slot, columns, input row x 8, output row x 8}; entries are numbered
 *   in the order of their first assignment; input row = a / topk in gu and a in dn, output row = a; unused columns and the
 *   entries behind the last run hold -1. The result is deterministic. */
int32_t tqmoe_dedup_maps(const int32_t * ids, const int32_t * slot_of, int32_t count, int32_t topk, int32_t * slots, int32_t * gu,
                         int32_t * dn, int32_t groups, void * stream, tqmoe_error * err);

/* -------------------------------------------------------------------------------------------------- banks
 * A bank is one projection of every expert: `experts` matrices of rows x cols stacked row-wise, expert e at row
 * e * rows (weight_format.hpp:61 "Stacked weights [experts * rows][cols]"); a non-owning view like tqllm::Mat
 * (weight_format.hpp:22-28). The library reads its own device layout, made from the raw GGUF block stream by
 * tqmoe_bank_load (the counterpart of WeightFormat::load, weight_format.hpp:41, and of the loaders in
 * src/formats/weight/q4.cpp:295-326, 495-530, 577-606, 802-836). Per 32 weights of a row (a sub-block):
 *   IQ4_XS  codes 16 B: byte j = weights j (low nibble) and j + 16 (high) of the sub-block (GGUF order);
 *           aux 8 B per 256 weights: GGUF's d (f16), scales_h, scales_l[4] repacked (the eight 6-bit scales minus 32 as
 *           signed 6-bit fields, d in the 16 bits between them). Rows are stored in tiles of 32: the 16 B
 *           of sub-block s of the 32 rows of a tile are contiguous (512 B), tiles of a row group follow each other by
 *           sub-block, and the 8 B records likewise (256 B per tile and super-block); rows must be a multiple of 32.
 *           The other formats are row-major (codes of a row contiguous, then its records).
 *   Q4_K    codes 16 B in the same nibble order; aux 16 B per 256 weights: d, dmin (f16), scales[12] as in GGUF.
 *   IQ3_S   codes 12 B: 8 lattice index bytes then 4 sign bytes; aux 16 B per 256 weights: d (f16), qh[8],
 *           scales[4], 2 B padding.
 *   NVFP4G  codes 16 B in the same nibble order (weights j and j + 16 of the sub-block); aux: one E4M3 scale per
 *           16 weights, [rows_total][cols / 16] bytes, then at the next multiple of 16 bytes rows_total fp32 globals
 *           (one per row; rows whose blocks disagree are rejected by the reference loader, q4.cpp:519-521, and by
 *           tqmoe_bank_load through *status).
 *   Q5_K    codes 16 B: the low four bits in the same nibble order; aux 48 B per 256 weights: d, dmin, scales[12] as in
 *           GGUF, then one 32-bit word per sub-block with the fifth bit of its weights (bit j = weight j).
 *   Q6_K    codes 24 B: 16 B of low nibbles in the same order, then 8 B with the upper two bits (byte k = weights
 *           4 k .. 4 k + 3); aux 32 B per 256 weights: the sixteen int8 scales in GGUF order (two per sub-block), d (f16),
 *           padding.
 *   IQ3_XXS codes 12 B: 8 lattice index bytes, then GGUF's word of four 7-bit sign fields and the 4-bit scale; aux 16 B per
 *           256 weights: d (f16), padding.
 *   IQ2_S   codes 12 B: 4 low index bytes, 4 sign bytes, the sub-block's qh byte, its scale byte, 2 B padding; aux as
 *           IQ3_XXS.
 *   IQ2_XS  codes 12 B: GGUF's four 16-bit fields (9-bit lattice index, 7 sign bits), the sub-block's scale byte, 3 B
 *           padding; aux as IQ3_XXS.
 *   IQ2_XXS codes 8 B: 4 lattice index bytes, then GGUF's word of four 7-bit sign fields and the 4-bit scale; aux as IQ3_XXS.
 *   Q3_K    codes 12 B: 8 B with the low two bits (byte k = weights 4 k .. 4 k + 3), then 4 B with the third bit (bit j =
 *           weight j; the weight is the three-bit value minus 4); aux 32 B per 256 weights: the sixteen 6-bit scales minus
 *           32 as int8 (two per sub-block), d (f16), padding.
 *   Q2_K    codes 8 B: two bits per weight (byte k = weights 4 k .. 4 k + 3); aux 32 B per 256 weights: GGUF's sixteen
 *           (scale | min << 4) bytes (two per sub-block), d, dmin (f16), padding.
 *   IQ1_S   codes 8 B: 4 low lattice index bytes, then GGUF's 16-bit qh of the sub-block (4 x 3 upper index bits, the 3-bit
 *           scale, the sign of the shift), 2 B padding; aux as IQ3_XXS.
 *   IQ4_NL  codes 16 B, GGUF's own nibble order; aux 2 B per sub-block: its d (f16).
 *   Q4_0    as IQ4_NL (the weight is the nibble minus 8).
 *   Q8_0    codes 32 B: the int8 values; aux 2 B per sub-block: its d (f16).
 * cols must be a multiple of 256 (128 for NVFP4G). Every format has the decode products and the fp16 grouped products
 * (tqmoe_expert_gemm, tqmoe_expert_gemm_gateup). The grouped int8 products take the formats with one scale per 32 weights
 * (IQ4_XS, IQ4_NL, IQ3_S, IQ3_XXS, IQ2_XXS, IQ2_XS, IQ2_S, IQ1_S, Q4_K, Q5_K, Q4_0, Q8_0), the grouped fp8 products NVFP4G;
 * Q6_K, Q3_K and Q2_K (a scale per 16 weights, half the depth of the int8 matrix instruction) have the fp16 grouped
 * products only. */
typedef struct tqmoe_bank {
    uint32_t struct_size;
    uint32_t type;            /* one of the bank formats of the enum above */
    int32_t experts;          /* matrices in the bank */
    int32_t rows, cols;       /* of one expert */
    const void * codes;       /* device, tqmoe_bank_layout's code_bytes */
    const void * aux;         /* device, tqmoe_bank_layout's aux_bytes */
} tqmoe_bank;

/* device bytes of the two planes for rows_total = experts * rows stacked rows */
int32_t tqmoe_bank_layout(uint32_t type, int64_t rows_total, int32_t cols, size_t * code_bytes, size_t * aux_bytes,
                          tqmoe_error * err);
/* gguf_blocks: device copy of the GGUF block stream of [rows_total][cols] (row-major, blocks of a row contiguous).
 * codes / aux: device outputs. status: optional device int32, set non-zero when a row's data is rejected. */
int32_t tqmoe_bank_load(uint32_t type, const void * gguf_blocks, int64_t rows_total, int32_t cols, void * codes,
                        void * aux, int32_t * status, void * stream, tqmoe_error * err);
/* rows [row0, row0 + nrows) of the stacked matrix as fp32 [nrows][cols]: the bank's decoded values, bit for bit those
 * of the reference's host decoder dequantize_host (src/formats/weight/dequant.cpp). Counterpart of
 * WeightFormat::dequant_rows_h (weight_format.hpp:84-86). */
int32_t tqmoe_bank_dequant(const tqmoe_bank * bank, int64_t row0, int64_t nrows, float * out, void * stream,
                           tqmoe_error * err);

/* ------------------------------------------------------------------------------------------ decode products
 * Activation image the decode products read: x = s * q with q = rint(x / s) held as two int8 planes
 * (q = 128 * hi + lo, 0 <= lo < 128, |q| <= 16383), so that integer dot products with the integer weight codes
 * reproduce the fp32 product to 2^-15 of the maximum the scale was taken from. tqmoe_quant_act and the top-k kernel
 * take one scale per row (s = amax of the row / 16383: the integer sums then run over whole 256-weight super-blocks);
 * tqmoe_expert_gateup writes its act rows with one scale per 32 values (amax of the block / 16383). Either way the
 * row stores a scale and a sum for every block. One image row is cols * 2 bytes of planes (64 B per 32 values: the hi
 * plane then the lo plane, each in the byte order of the banks' code bytes), then cols / 32 fp32 scales, then
 * cols / 32 fp32 sums of q * s; tqmoe_act_image_bytes gives the size for n rows. The image is private to the library:
 * only tqmoe_quant_act, the top-k kernel of tqmoe_layer_forward and tqmoe_expert_gateup write it, only the decode
 * products read it. */
size_t  tqmoe_act_image_bytes(int32_t n, int32_t cols);
int32_t tqmoe_quant_act(const void * x, uint32_t xtype, int32_t n, int32_t cols, void * image, void * stream,
                        tqmoe_error * err);

/* y[a][r] = sum_c W[ids[a] * rows + r][c] * x[row(a)][c], a < n * topk, row(a) = a (per_expert_input) or a / topk.
 * image: activation image of the input rows; y: device [n * topk][rows] of ytype (F32 or BF16).
 * Replaces WeightFormat::expert_matvec (weight_format.hpp:62-64, src/formats/weight/quant.cu:69-111). */
int32_t tqmoe_expert_matvec(const tqmoe_bank * bank, const void * image, void * y, uint32_t ytype, const int32_t * ids,
                            int32_t n, int32_t topk, int32_t per_expert_input, void * stream, tqmoe_error * err);
/* gate and up over the same ids in one launch (WeightFormat::expert_matvec2, weight_format.hpp:70-73) */
int32_t tqmoe_expert_matvec2(const tqmoe_bank * gate, const tqmoe_bank * up, const void * image, void * y_gate,
                             void * y_up, uint32_t ytype, const int32_t * ids, int32_t n, int32_t topk, void * stream,
                             tqmoe_error * err);

/* The same two products on the rows the reference's callers hold (fp16 rows; any of F32 / F16 / BF16 here): exactly
 * WeightFormat::expert_matvec(const Mat &, const __half * x, bf16 * y, int rows, const int * ids, int n, int topk,
 * bool per_expert_input, stream) and expert_matvec2 (weight_format.hpp:62-64, 70-73). x: device [n][cols], or
 * [n * topk][cols] with per_expert_input. The activation image is made in `scratch` (caller-owned device memory of
 * tqmoe_act_image_bytes(input rows, cols); one enqueue order: image, then product) and is dead after the call. */
int32_t tqmoe_expert_matvec_rows(const tqmoe_bank * bank, const void * x, uint32_t xtype, void * y, uint32_t ytype,
                                 const int32_t * ids, int32_t n, int32_t topk, int32_t per_expert_input, void * scratch,
                                 size_t scratch_bytes, void * stream, tqmoe_error * err);
int32_t tqmoe_expert_matvec2_rows(const tqmoe_bank * gate, const tqmoe_bank * up, const void * x, uint32_t xtype,
                                  void * y_gate, void * y_up, uint32_t ytype, const int32_t * ids, int32_t n, int32_t topk,
                                  void * scratch, size_t scratch_bytes, void * stream, tqmoe_error * err);

/* The same products over the decode grouping maps of tqmoe_dedup_maps (kDedupStride = 18 ints a group: slot, columns, input
 * row x 8, output row x 8): y[output row][r] = sum_c W[slot * rows + r][c] * x[input row][c] for every column of every group
 * whose slot is not negative. WeightFormat::expert_matvec_dedup / expert_matvec_dedup2 (weight_format.hpp:66-69; kernels
 * src/formats/weight/quant.cu:113-129, 196-205, quant_u4h.inc:437-447, 488-491). bank2 / y2: a second bank of the same format
 * and shape over the same maps (gate and up), or NULL. x: device rows of xtype; y: device rows of bank rows elements of ytype
 * (F32 or BF16); rows no column names stay untouched. The map's columns run as assignments of the decode kernels (which read an
 * expert's weights once for all of them); scratch: device memory of tqmoe_expert_matvec_dedup_scratch_bytes(), dead after
 * the call. groups * 8 <= 65535. */
size_t  tqmoe_expert_matvec_dedup_scratch_bytes(int32_t groups, int32_t rows, int32_t cols, uint32_t ytype, int32_t two_banks);
int32_t tqmoe_expert_matvec_dedup(const tqmoe_bank * bank, const tqmoe_bank * bank2, const void * x, uint32_t xtype, void * y,
                                  void * y2, uint32_t ytype, const int32_t * dmap, int32_t groups, void * scratch,
                                  size_t scratch_bytes, void * stream, tqmoe_error * err);

/* Decode stages of the layer (tqmoe_layer_forward is router, top-k, tqmoe_extend_ids, tqmoe_quant_act, these two and
 * tqmoe_combine_strided). `ids` holds the expert of every (token, slot), [n][slots]: the routed ids and, when
 * slots == topk + 1, the shared expert's bank index in the last slot (tqmoe_extend_ids makes it). One block serves every
 * assignment of its expert, so a step reads each distinct expert's weights from HBM once.
 *
 * tqmoe_extend_ids: out[t][s] = s < topk ? ids[t][s] : extra. tqllm_cuda::moe_extend_ids without slot maps
 * (src/experts/moe_kernels.cuh:77-78, moe.cu:204-216).
 * tqmoe_expert_gateup: act[a] = silu(gate_e x[t]) * (up_e x[t]) for a = t * slots + s, written as an activation image of
 * n * slots rows of gate->rows values; a shared assignment (s >= topk) only has its first shared_ff values.
 * Counterpart of WeightFormat::expert_gemm_gateup (weight_format.hpp:57-59: gate and up in one launch with the SwiGLU
 * epilogue) at decode sizes.
 * tqmoe_expert_down: y[a] = down_e act[a], fp32 [n * slots][down->rows]; a shared assignment reads the first shared_ff
 * columns. WeightFormat::expert_matvec with per_expert_input (weight_format.hpp:62-64). */
int32_t tqmoe_extend_ids(const int32_t * ids, int32_t * out, int32_t topk, int32_t n, int32_t extra, void * stream,
                         tqmoe_error * err);
int32_t tqmoe_expert_gateup(const tqmoe_bank * gate, const tqmoe_bank * up, const void * x_image, void * act_image,
                            const int32_t * ids, int32_t n, int32_t slots, int32_t topk, int32_t shared_ff,
                            void * stream, tqmoe_error * err);
int32_t tqmoe_expert_down(const tqmoe_bank * down, const void * act_image, float * y, const int32_t * ids, int32_t n,
                          int32_t slots, int32_t topk, int32_t shared_ff, void * stream, tqmoe_error * err);

/* act[i] = silu(gate[i]) * up[i], fp32 in and out (the reference's moe_swiglu, moe_kernels.cuh:71-72, rounds its
 * bf16 inputs' product through bf16 to fp16; here nothing is rounded below fp32). */
int32_t tqmoe_swiglu(const float * gate, const float * up, float * act, int64_t count, void * stream, tqmoe_error * err);
/* the same with the reference's optional clamp (MoeConfig::swiglu_clamp, src/experts/moe.hpp:34-36; moe_expert_ffn,
 * src/experts/moe.cpp:128-143): swiglu_clamp <= 1e-6: none; else up goes to [-swiglu_clamp, swiglu_clamp] and either the gate
 * to at most swiglu_clamp before the activation (clamp_gate nonzero) or silu(gate) to at most swiglu_clamp after it. */
int32_t tqmoe_swiglu_clamped(const float * gate, const float * up, float * act, int64_t count, float swiglu_clamp, int32_t clamp_gate,
                             void * stream, tqmoe_error * err);

/* out[t][j] = sum_s weights[t][s] * routed[t * topk + s][j] (s ascending) + shared_weights[t] * shared[t][j];
 * routed / shared fp32, shared and shared_weights may be NULL together; out of otype (F32 or BF16).
 * Replaces tqllm_cuda::moe_sum (moe_kernels.cuh:73-74, moe.cu:224-234) and fn_moe_combine (qwen4exp.cu:846-851);
 * host meaning: moe_combine (src/experts/moe.cpp:157-163). No atomics: the sum order is fixed. */
int32_t tqmoe_combine(const float * routed, const float * shared, const float * weights, const float * shared_weights,
                      void * out, uint32_t otype, int32_t hidden, int32_t topk, int32_t n, void * stream,
                      tqmoe_error * err);
/* the same with `slots` routed rows per token (the first topk weighted) and the shared rows shared_ld floats apart:
 * tqllm_cuda::moe_sum_strided (moe_kernels.cuh:80-81, moe.cu:197-210). hidden and shared_ld multiples of 4. */
int32_t tqmoe_combine_strided(const float * routed, int32_t slots, const float * shared, int64_t shared_ld,
                              const float * weights, const float * shared_weights, void * out, uint32_t otype,
                              int32_t hidden, int32_t topk, int32_t n, void * stream, tqmoe_error * err);

/* ------------------------------------------------------------------------------------------ prefill products
 * Grouped int8 x int8 -> int32 products on the matrix cores over the dispatch lists: IQ4_XS, IQ4_NL, IQ3_S, IQ3_XXS,
 * IQ2_XXS, IQ2_XS, IQ2_S, IQ1_S and Q4_K banks, with exact weights (the reference's int8 path covers its u4h formats the same way,
 * quant_u4h.inc:783-789, 839-845, and its MMQ path the IQ formats, mmq_experts.cu:193-196). Rows a multiple of 32,
 * columns of 256.
 * counts / offsets / perm are tqmoe_dispatch's lists over ids [n][slots] with `experts` = the banks' experts.
 *
 * tqmoe_quant_rows_i8: per input row q = rint(x * 127 / amax), scale = amax / 127 (0 for a zero row): the per-token mode
 * of the reference's activation quantiser k_quant_act_rows (src/formats/weight/quant_kernels.cuh:17-19, mode 2;
 * quant_u4h.inc:790-820). q: device int8 [rows][cols], every 32 values in the byte order of the banks' code bytes;
 * scale: device fp32 [rows]. cols a multiple of 32.
 * tqmoe_group_rows_i8: the same quantiser applied to the input row (a / xdiv) of every listed assignment a, the rows
 * gathered expert by expert into tiles of 32 (every expert padded to whole tiles) in the operand order of the matrix
 * instruction: the form the two products below read. q: device int8 [tqmoe_grouped_rows()][cols], scale: device, 4 bytes
 * x tqmoe_grouped_scale_words() (the fp32 row scales, then the library's index of the tiles); the layout is private to
 * the library. xdiv = slots for the layer input (row = token), 1 for
 * rows that exist per assignment. This is the step the reference does with mmq_quantize_act_rows
 * (src/experts/mmq_experts.cu:79-95: quantise and arrange the rows of every expert tile).
 * tqmoe_gather_rows_i8: the arranging alone, from rows tqmoe_quant_rows_i8 has quantised (rows_q [rows][cols], rows_scale
 * [rows]): the same q / scale as tqmoe_group_rows_i8 on the unquantised rows, bit for bit, with every input row
 * quantised once however many assignments read it (the layer input: xdiv = slots).
 * tqmoe_expert_gemm_gateup_i8: act[a] = silu(gate_e x) * (up_e x) as fp16 [n * slots][gate->rows] for every listed
 * assignment a = t * slots + s. WeightFormat::expert_gemm_gateup (weight_format.hpp:57-59) with the int8 operands of
 * expert_gemm_i8 (weight_format.hpp:54-56).
 * tqmoe_expert_gemm_i8: y[a] = W_e x[a] as fp16 [n * slots][bank->rows]. WeightFormat::expert_gemm_i8, mode 2
 * (per-token scales). xq / xs: tqmoe_group_rows_i8's outputs for the same lists.
 * Assignments of the bank's last expert use only shared_lim rows (gate / up; the rest of their act row is zero) or columns
 * (down) when slots > topk (the shared expert); shared_lim a multiple of 256. Rows of assignments that are in no list
 * stay untouched. The products hand their work out through counters that live behind the grouped rows' scales (zero
 * between launches: the grouping call clears them and every product launch leaves them cleared), so two products over
 * the same grouped rows may follow each other on a stream, also in a replayed graph, but must not run at the same
 * time. */
int32_t tqmoe_quant_rows_i8(const void * x, uint32_t xtype, int64_t rows, int32_t cols, int8_t * q, float * scale,
                            void * stream, tqmoe_error * err);
int64_t tqmoe_grouped_rows(int64_t assignments, int32_t experts);
int64_t tqmoe_grouped_scale_words(int64_t assignments, int32_t experts);
int32_t tqmoe_group_rows_i8(const void * x, uint32_t xtype, int32_t cols, const int32_t * counts, const int32_t * offsets,
                            const int32_t * perm, int32_t experts, int64_t assignments, int32_t xdiv, int8_t * q,
                            float * scale, void * stream, tqmoe_error * err);
int32_t tqmoe_gather_rows_i8(const int8_t * rows_q, const float * rows_scale, int32_t cols, const int32_t * counts,
                             const int32_t * offsets, const int32_t * perm, int32_t experts, int64_t assignments,
                             int32_t xdiv, int8_t * q, float * scale, void * stream, tqmoe_error * err);
int32_t tqmoe_expert_gemm_gateup_i8(const tqmoe_bank * gate, const tqmoe_bank * up, const int8_t * xq, const float * xs,
                                    const int32_t * counts, const int32_t * offsets, const int32_t * perm, int32_t n,
                                    int32_t slots, int32_t topk, int32_t shared_lim, void * act_f16, void * stream,
                                    tqmoe_error * err);
int32_t tqmoe_expert_gemm_i8(const tqmoe_bank * bank, const int8_t * xq, const float * xs, const int32_t * counts,
                             const int32_t * offsets, const int32_t * perm, int32_t n, int32_t slots, int32_t topk,
                             int32_t shared_lim, void * y_f16, void * stream, tqmoe_error * err);
/* The same steps with a scale per 32 values of every input row in place of one per row: the per-32-block mode of the
 * reference's activation quantiser and of expert_gemm_i8 (k_quant_act_rows / k_expert_gemm_i8 mode 1,
 * src/formats/weight/quant_kernels.cuh:13-19; quant_act_rows_k<false> and u4h_i8_gemm_k<.., TOKEN = false>,
 * quant_u4h.inc:790-822, 849-935), which isolates an outlier to its block. A block's product is an exact integer sum
 * that is scaled by the weights' scale and the row's block scale before it joins the fp32 result, as in the reference.
 * tqmoe_quant_rows_i8_blocks: q as tqmoe_quant_rows_i8, scales fp32 [rows][cols / 32] (amax of the block / 127), qsum
 * int16 [rows][cols / 32][2] = the sums of q over each 16 values (the reference's xsum; may be null: the products here
 * take the weights' minimum term from a matrix product of their own and do not read it).
 * tqmoe_group_rows_i8_blocks / tqmoe_gather_rows_i8_blocks: q / scale as above (every row scale 1) and block_scale, device
 * fp32, tqmoe_grouped_block_scale_words(assignments, experts, cols) words ([row tile][cols / 32][32 rows]).
 * tqmoe_expert_gemm_gateup_i8_blocks / tqmoe_expert_gemm_i8_blocks: the two products on such rows; int8 formats only. */
int32_t tqmoe_quant_rows_i8_blocks(const void * x, uint32_t xtype, int64_t rows, int32_t cols, int8_t * q, float * scales,
                                   int16_t * qsum, void * stream, tqmoe_error * err);
int64_t tqmoe_grouped_block_scale_words(int64_t assignments, int32_t experts, int32_t cols);
int32_t tqmoe_group_rows_i8_blocks(const void * x, uint32_t xtype, int32_t cols, const int32_t * counts,
                                   const int32_t * offsets, const int32_t * perm, int32_t experts, int64_t assignments,
                                   int32_t xdiv, int8_t * q, float * scale, float * block_scale, void * stream,
                                   tqmoe_error * err);
int32_t tqmoe_gather_rows_i8_blocks(const int8_t * rows_q, const float * rows_scales, int32_t cols, const int32_t * counts,
                                    const int32_t * offsets, const int32_t * perm, int32_t experts, int64_t assignments,
                                    int32_t xdiv, int8_t * q, float * scale, float * block_scale, void * stream,
                                    tqmoe_error * err);
int32_t tqmoe_expert_gemm_gateup_i8_blocks(const tqmoe_bank * gate, const tqmoe_bank * up, const int8_t * xq,
                                           const float * xs, const float * block_scale, const int32_t * counts,
                                           const int32_t * offsets, const int32_t * perm, int32_t n, int32_t slots,
                                           int32_t topk, int32_t shared_lim, void * act_f16, void * stream,
                                           tqmoe_error * err);
int32_t tqmoe_expert_gemm_i8_blocks(const tqmoe_bank * bank, const int8_t * xq, const float * xs, const float * block_scale,
                                    const int32_t * counts, const int32_t * offsets, const int32_t * perm, int32_t n,
                                    int32_t slots, int32_t topk, int32_t shared_lim, void * y_f16, void * stream,
                                    tqmoe_error * err);
/* The E4M3 form of the same steps for NVFP4G banks (fp8 x fp8 -> fp32 on the matrix cores): the input rows as E4M3 with
 * one scale per row, amax / 448 (the reference's fp8_quant_rows, src/core/fp8_gemm.cuh:19-31: scales applied after the
 * product); the weights widened to E4M3 bytes, e2m1 * (E4M3 scale of the 16 weights) / 8 rounded to nearest even (a
 * declared lossy operand: up to six significant bits into four; the 8 keeps 6 * 448 inside the format), 8 * the row's
 * fp32 global applied to the result. q: E4M3 bytes in the layout of tqmoe_group_rows_i8's; tqmoe_gather_rows_i8 arranges rows that
 * tqmoe_quant_rows_fp8 has quantised (it copies bytes). Rows a multiple of 32, columns of 256. */
int32_t tqmoe_quant_rows_fp8(const void * x, uint32_t xtype, int64_t rows, int32_t cols, uint8_t * q, float * scale,
                             void * stream, tqmoe_error * err);
int32_t tqmoe_group_rows_fp8(const void * x, uint32_t xtype, int32_t cols, const int32_t * counts, const int32_t * offsets,
                             const int32_t * perm, int32_t experts, int64_t assignments, int32_t xdiv, uint8_t * q,
                             float * scale, void * stream, tqmoe_error * err);
int32_t tqmoe_expert_gemm_gateup_fp8(const tqmoe_bank * gate, const tqmoe_bank * up, const uint8_t * xq, const float * xs,
                                     const int32_t * counts, const int32_t * offsets, const int32_t * perm, int32_t n,
                                     int32_t slots, int32_t topk, int32_t shared_lim, void * act_f16, void * stream,
                                     tqmoe_error * err);
int32_t tqmoe_expert_gemm_fp8(const tqmoe_bank * bank, const uint8_t * xq, const float * xs, const int32_t * counts,
                              const int32_t * offsets, const int32_t * perm, int32_t n, int32_t slots, int32_t topk,
                              int32_t shared_lim, void * y_f16, void * stream, tqmoe_error * err);
/* The same two products for every bank format, with fp16 operands (weights decoded and rounded to fp16, input rows
 * converted to fp16, fp32 accumulation on the matrix cores): WeightFormat::expert_gemm (weight_format.hpp:51-53) and
 * expert_gemm_gateup (weight_format.hpp:57-59). x: device rows of xtype with the bank's cols; the input row of
 * assignment a is a / slots (tqmoe_expert_gemm_gateup; tqmoe_expert_gemm without per_expert_input) or a itself
 * (per_expert_input). shared_lim a multiple of 32. act: fp16 [n * slots][rows]; y: [n * slots][rows] of ytype (F16, BF16 or F32).
 * n * slots only bounds the number of listed assignments (it sizes the launch): any upper bound will do. */
int32_t tqmoe_expert_gemm_gateup(const tqmoe_bank * gate, const tqmoe_bank * up, const void * x, uint32_t xtype,
                                 const int32_t * counts, const int32_t * offsets, const int32_t * perm, int32_t n,
                                 int32_t slots, int32_t topk, int32_t shared_lim, void * act_f16, void * stream,
                                 tqmoe_error * err);
int32_t tqmoe_expert_gemm(const tqmoe_bank * bank, const void * x, uint32_t xtype, const int32_t * counts,
                          const int32_t * offsets, const int32_t * perm, int32_t n, int32_t slots, int32_t topk,
                          int32_t shared_lim, int32_t per_expert_input, void * y, uint32_t ytype, void * stream,
                          tqmoe_error * err);
/* The reference's form of the dispatch lists, counts [experts] + groups [experts][capacity] (what its grouped products
 * take: weight_format.hpp:51-59; filled by moe_group, moe.cu:168-176, or on the host, prefill_plan.hpp:63-74), as the
 * lists the grouped products above read: offsets [experts + 1] = exclusive scan of min(counts, capacity), perm = the
 * experts' lists one behind the other (perm needs room for the sum of the counts; experts * capacity always suffices).
 * The order inside an expert is kept; the products do not depend on it. */
int32_t tqmoe_lists_from_groups(const int32_t * counts, const int32_t * groups, int32_t capacity, int32_t experts,
                                int32_t * offsets, int32_t * perm, void * stream, tqmoe_error * err);
/* The same, and counts_out [experts] = min(counts, capacity): the counts the grouped products must be given with these lists
 * (with the caller's own counts an expert whose count exceeds the capacity would run past its span of perm). */
int32_t tqmoe_lists_from_groups_clamped(const int32_t * counts, const int32_t * groups, int32_t capacity, int32_t experts,
                                        int32_t * counts_out, int32_t * offsets, int32_t * perm, void * stream, tqmoe_error * err);

/* WeightFormat::expert_gemm_i8 with the reference's own operands (weight_format.hpp:54-56; called from
 * src/models/qwen/qwen4exp/fn_prefill.cpp:192-194 on the rows k_quant_act_rows leaves, quant_kernels.cuh:13-19):
 *   xq    device int8 [input rows][cols], natural order;
 *   xs    device fp32 [input rows][cols / 32]: mode 1 the blocks' scales, mode 2 the token's scale in every entry ([row][0] is read);
 *   xsum  the reference's int16 sums per 16 values: not read (may be NULL);
 *   counts [experts], groups [experts][capacity]: the reference's lists of assignment indices a; input row a / topk, or a with
 *   per_expert_input; experts must be the bank's;
 *   y     device [assignments][bank rows] of ytype (BF16 as the reference, or F16); rows of unlisted assignments stay untouched.
 * One call enqueues the list conversion, the arranging of the rows into the operand tiles and the product.
 * max_assignments bounds the listed assignments (n * topk of the pass); scratch: device memory of
 * tqmoe_expert_gemm_i8_ref_scratch_bytes(experts, max_assignments, cols, mode), dead after the call.
 * TQMOE_E_UNSUPPORTED (the base class's `false`): no int8 grouped product for the bank's format. */
size_t  tqmoe_expert_gemm_i8_ref_scratch_bytes(int32_t experts, int64_t max_assignments, int32_t cols, int32_t mode);
int32_t tqmoe_expert_gemm_i8_ref(const tqmoe_bank * bank, const int8_t * xq, const float * xs, const int16_t * xsum, void * y, uint32_t ytype,
                                 const int32_t * counts, const int32_t * groups, int32_t capacity, int32_t experts, int32_t topk,
                                 int32_t per_expert_input, int32_t mode, int64_t max_assignments, void * scratch, size_t scratch_bytes,
                                 void * stream, tqmoe_error * err);

/* tqmoe_combine_strided with fp16 rows (the prefill products' output) */
int32_t tqmoe_combine_strided_f16(const void * routed, int32_t slots, const void * shared, int64_t shared_ld,
                                  const float * weights, const float * shared_weights, void * out, uint32_t otype,
                                  int32_t hidden, int32_t topk, int32_t n, void * stream, tqmoe_error * err);

/* tqmoe_combine_strided with the residual stream added: out = bf16(bf16(sum) + residual), the two roundings of the
 * reference's moe_sum into bf16 followed by add_sumsq (src/models/qwen/qwen35/qwen35_forward.cpp:1248-1250,
 * src/formats/weight/quant_tq3.inc:303-313). routed / shared: F32 or F16 rows (rtype); residual, out: device
 * [n][hidden] bf16. out may be the residual buffer itself (every element is read before it is written). */
int32_t tqmoe_combine_residual(const void * routed, uint32_t rtype, int32_t slots, const void * shared, int64_t shared_ld,
                               const float * weights, const float * shared_weights, const void * residual, void * out,
                               int32_t hidden, int32_t topk, int32_t n, void * stream, tqmoe_error * err);

/* ------------------------------------------------------------------------------------- the step before the layer
 * Residual add and RMS norm of the rows the router and the experts read, one launch for the reference's pair
 * add_sumsq + norm_h (Qwen35Engine::ffn_block, qwen35_forward.cpp:1114-1115; quant_tq3.inc:303-313, quant.cu:647-661):
 *   rows[t][i]   = bf16(rows[t][i] + residual[t][i])            in place; skipped when residual is NULL
 *   normed[t][i] = bf16((rows[t][i] * inv_t) * weight[i]),      inv_t = 1 / sqrt(mean_i rows[t][i]^2 + eps)
 * rows, residual: device [n][hidden] bf16; weight: device [hidden] fp32; normed: device [n][hidden] of ntype (BF16,
 * or F16 holding the bf16-rounded value as the reference's fp16 activations do). hidden % 8 == 0. The sum of squares
 * is accumulated in fp32 in this kernel's own order: normed values can differ from the reference's by one bf16 step
 * where they sit on a rounding boundary; the updated rows are bit-exact. */
int32_t tqmoe_add_rmsnorm(void * rows, const void * residual, const float * weight, float eps, void * normed,
                          uint32_t ntype, int32_t hidden, int32_t n, void * stream, tqmoe_error * err);

/* ---------------------------------------------------------------------------------------------- whole layer
 * hidden states + router weights + expert banks in, combined hidden states out: the sequence of
 * Qwen35Engine::ffn_block steps 2-9 (src/models/qwen/qwen35/qwen35_forward.cpp:1123-1248) and of the Flash-Next
 * layer (src/models/qwen/qwen4exp/fn_layer_forward.cpp:311-336, 447-520) in one call.
 * The shared expert, when has_shared, is expert index n_expert of the three banks (so banks hold n_expert + 1
 * matrices), uses the first shared_ff rows of gate / up and the first shared_ff columns of down, and is weighted by
 * sigmoid(router logit column n_expert), or by 1 when shared_gate is NULL (an always-on shared expert without a gate row).
 * MoeConfig::swiglu_clamp (src/experts/moe.hpp:34-36) and the clamp_gate switch of moe_expert_ffn (src/experts/moe.cpp:115-143)
 * are the descriptor's last two fields. */
typedef struct tqmoe_layer {
    uint32_t struct_size;
    int32_t hidden, ff, n_expert, topk;
    int32_t has_shared, shared_ff;
    float weight_scale;               /* 0 or 1: none */
    const void * router;              /* device [n_expert][hidden] of router_type */
    const void * shared_gate;         /* device [hidden] of router_type, or NULL */
    uint32_t router_type;             /* TQMOE_F32 or TQMOE_BF16 */
    tqmoe_bank gate, up, down;        /* gate / up: rows ff, cols hidden; down: rows hidden, cols ff */
    /* Routing mode, as tqmoe_topk_gated takes it. A descriptor whose struct_size ends before these fields, or that
     * leaves them zero, routes by softmax with normalised weights and no bias. */
    int32_t gating;                   /* 0: softmax, else a TQMOE_GATE_ value */
    int32_t raw_weights;              /* nonzero: the selected weights are not normalised */
    const float * probs_bias;         /* device [n_expert] fp32 selection bias, or NULL */
    /* The reference's TQFN_PREFILL_INT8 (fn_prefill.cpp:100). 0 (or a descriptor that ends before this field): the library
     * picks the grouped products of a prefill-sized batch, the 8-bit ones (a scale per token) where they are the faster ones
     * for the banks' formats and the batch, else the fp16 ones. 1: the int8 grouped products with one scale per 32
     * activations (its value 1). 2: the int8 grouped products with one scale per token (its value 2). 1 and 2 apply where
     * both banks' formats have int8 grouped products; NVFP4G banks (fp8 products) and the decode kernels ignore the field. */
    int32_t act_blocks;
    /* Clamp of the SwiGLU inputs, applied in the fused gate / up epilogues of every path (routed and shared experts alike).
     * swiglu_clamp <= 1e-6 (or a descriptor that ends before this field): none. Else up is clamped to
     * [-swiglu_clamp, swiglu_clamp] and either the gate to at most swiglu_clamp before the activation (clamp_gate nonzero:
     * the GLM branch) or silu(gate) to at most swiglu_clamp after it (clamp_gate zero), as moe_expert_ffn does. */
    float swiglu_clamp;
    int32_t clamp_gate;
} tqmoe_layer;

size_t  tqmoe_layer_workspace_bytes(const tqmoe_layer * layer, int32_t n);
/* Which expert products tqmoe_layer_forward runs for n tokens of this layer (the choice depends on the batch and the
 * bank formats only, never on the data, so that a token's result does not depend on what else is routed; the reference
 * makes its switch slot-independent for the same reason, src/models/qwen/qwen4exp/fn_layer_forward.cpp:408-414):
 * the decode kernels (one read of every distinct expert), the grouped 8-bit products, or the grouped fp16 products.
 * With act_blocks zero the grouped products are the ones measured faster for the formats: int8 for IQ4_XS from 1024
 * tokens, for Q4_K from 2048 and for the two- and three-bit lattice formats, fp8 for NVFP4G, fp16 otherwise.
 * Negative: the descriptor is invalid. */
enum { TQMOE_PATH_DECODE = 0, TQMOE_PATH_GROUPED_I8 = 1, TQMOE_PATH_GROUPED_F16 = 2, TQMOE_PATH_GROUPED_FP8 = 3 };
int32_t tqmoe_layer_path(const tqmoe_layer * layer, int32_t n);
/* x: device [n][hidden] of xtype; out: device [n][hidden] of otype (F32 or BF16); ids_out [n][topk], weights_out
 * [n][topk], logits_out [n][n_expert + 1] optional device outputs (NULL to skip). */
int32_t tqmoe_layer_forward(const tqmoe_layer * layer, const void * x, uint32_t xtype, int32_t n, void * out,
                            uint32_t otype, int32_t * ids_out, float * weights_out, float * logits_out,
                            void * workspace, size_t workspace_bytes, void * stream, tqmoe_error * err);

/* tqmoe_layer_forward with the residual stream added to the result: out[t] = bf16(bf16(layer(x)[t]) + residual[t]), the
 * add that follows the layer in the reference (qwen35_forward.cpp:1250). residual, out: device [n][hidden] bf16; out may
 * be the residual buffer. */
int32_t tqmoe_layer_forward_residual(const tqmoe_layer * layer, const void * x, uint32_t xtype, const void * residual,
                                     int32_t n, void * out, int32_t * ids_out, float * weights_out, float * logits_out,
                                     void * workspace, size_t workspace_bytes, void * stream, tqmoe_error * err);

#ifdef __cplusplus
}
#endif
#endif

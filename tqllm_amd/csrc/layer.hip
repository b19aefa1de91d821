// The whole layer behind one entry point: router -> top-k -> activation image -> gate/up + SwiGLU -> down + combine.
#include <algorithm>

#include "formats.cuh"

namespace tqmoe {
int32_t check_bank(const tqmoe_bank * b, const char * what, tqmoe_error * err);
int32_t enqueue_topk(const float * logits, int32_t * ids, float * weights, float * shared_weights, int32_t * ext_ids, int32_t extra, const void * x,
                     uint32_t xtype, int32_t cols, void * image, int32_t experts, int32_t topk, int32_t n, float scale, int32_t gating,
                     const float * bias, int32_t norm, hipStream_t s, int32_t shared_ungated);
bool plane_gemm_has(uint32_t type);
bool plane_gemm_is_fp8(uint32_t type);
// decode.hip: the gate / up products with the clamp of the SwiGLU inputs
int32_t expert_gateup_glu(const tqmoe_bank * gate, const tqmoe_bank * up, const void * x_image, void * act_image, const int32_t * ids, int32_t n,
                          int32_t slots, int32_t topk, int32_t shared_ff, Glu glu, void * stream, tqmoe_error * err);
int32_t gemm_8bit_common(const tqmoe_bank * b0, const tqmoe_bank * b1, const int8_t * xq, const float * xs, const int32_t * counts, const int32_t * offsets,
                         const int32_t * perm, int32_t n, int32_t slots, int32_t topk, int32_t shared_lim, void * out, int gateup, void * stream,
                         tqmoe_error * err, const char * what, bool fp8, const float * block_scale, bool blocks, Glu glu, int out_bf16, const float * plan_from);
// the act rows' grouping and the down product read the index that the input rows' grouping built (the same lists)
int32_t group_rows_common(const void * x, uint32_t xtype, int32_t cols, const int32_t * counts, const int32_t * offsets, const int32_t * perm, int32_t experts,
                          int64_t assignments, int32_t xdiv, void * q, float * scale, void * stream, tqmoe_error * err, bool f8, const char * what,
                          float * block_scale, bool blocks, const float * plan_from);
int32_t gemm_f16_common(const tqmoe_bank * b0, const tqmoe_bank * b1, const void * x, uint32_t xtype, const int32_t * counts, const int32_t * offsets,
                        const int32_t * perm, int32_t n, int32_t slots, int32_t topk, int32_t shared_lim, int32_t xdiv, void * out, uint32_t otype, int gateup,
                        void * stream, tqmoe_error * err, const char * what, Glu glu);

namespace {

// Where the descriptor asks for the int8 grouped products (act_blocks nonzero), IQ4_XS banks take them from kGroupedMin tokens.
constexpr int kGroupedMin = 64;
// Left to the library (act_blocks zero), IQ4_XS banks take them from kInt8Tokens tokens: measured at 512 experts, top-10, on
// uniform and on Zipf routing, the fp16 grouped products are level or up to a fifth faster below (most experts then hold a
// row tile or two, which the fp16 kernel's one-expert blocks serve better), the int8 products a seventh faster at 4096.
constexpr int kInt8Tokens = 1024;
constexpr int kDecodeAssignments = 65535;   // per decode launch
constexpr int kDecodeDedup = 2048;          // assignments up to which the decode kernels serve an expert's rows together
constexpr int kGroupedPerBank = 3;          // assignments per expert from which the fp16 grouped products are the faster path

struct Plan {  // byte offsets into the workspace
    bool grouped;   // the grouped products (prefill sizes): int8 for IQ4_XS banks, fp16 for the other formats
    bool int8;
    int chunk;   // tokens per pass of the expert stages
    size_t logits, ids, weights, shared_w, ids_ext, total;
    size_t ximage, aimage, y;                                                // decode path
    size_t xq, xs, counts, offsets, perm, dispatch_ws, act16, aq, as, y16, rq, rs;   // grouped path
    bool blocks;            // int8 products with a scale per 32 activations
    size_t xbs, abks;        // their block scales
};

// the 8-bit grouped products: both banks' formats have one with the same operand type (int8, or E4M3 for NVFP4G)
bool int8_ok(const tqmoe_layer & L) {
    return plane_gemm_has(L.gate.type) && plane_gemm_has(L.down.type) && plane_gemm_is_fp8(L.gate.type) == plane_gemm_is_fp8(L.down.type) &&
           L.hidden % 256 == 0 && L.ff % 256 == 0 && (!L.has_shared || L.shared_ff % 256 == 0);
}

// The descriptor grew three times: one that ends before the routing fields means softmax, normalised, no bias; one that
// ends before act_blocks means a scale per token; one that ends before swiglu_clamp means no clamp.
constexpr size_t kLayerBaseSize = offsetof(tqmoe_layer, gating), kLayerRoutingSize = offsetof(tqmoe_layer, act_blocks);
constexpr size_t kLayerBlocksSize = offsetof(tqmoe_layer, swiglu_clamp);
// the descriptor's request for the int8 grouped products: 0 none (the library chooses), 1 a scale per 32 activations, 2 a scale per token
int int8_mode_of(const tqmoe_layer & L) { return L.struct_size >= kLayerBlocksSize ? (L.act_blocks == 1 ? 1 : L.act_blocks == 2 ? 2 : 0) : 0; }
bool act_blocks_of(const tqmoe_layer & L) { return int8_mode_of(L) == 1; }
// Formats whose 8-bit grouped products are the faster ones at n tokens (measured against the fp16 grouped products at 256
// experts top-8 and at 64 experts top-8, 256 to 4096 tokens, uniform and Zipf routing): the lattice formats of two and three
// bits (a tenth faster), NVFP4G on its fp8 products, IQ4_XS from kInt8Tokens tokens, Q4_K from 2048 tokens (with fp32 input
// rows, which the fp16 kernel converts block by block, int8 is a tenth faster there; with 16-bit rows the two are level).
// IQ3_S, Q5_K, IQ4_NL, Q4_0 and Q8_0 run 5 to 25 % faster on the fp16 products (their row-major codes reach the int8 kernel's
// lanes in 8-byte pieces of 32 different rows, and two int8 planes cost the matrix pipe what one fp16 operand does).
bool int8_faster(uint32_t type, int n) {
    switch (type) {
        case TQMOE_IQ4_XS: return n >= kInt8Tokens;
        case TQMOE_Q4_K: return n >= 2 * kInt8Tokens;
        case TQMOE_NVFP4G: case TQMOE_IQ3_XXS: case TQMOE_IQ2_XXS: case TQMOE_IQ2_XS: case TQMOE_IQ2_S: case TQMOE_IQ1_S: return true;
        default: return false;
    }
}
// a descriptor that ends before swiglu_clamp does not clamp
Glu glu_of(const tqmoe_layer & L) { return L.struct_size >= sizeof(tqmoe_layer) ? Glu{L.swiglu_clamp, L.clamp_gate ? 1 : 0} : Glu{0.f, 0}; }

Plan plan_for(const tqmoe_layer & L, int n) {
    Plan p{};
    const int slots = L.topk + (L.has_shared ? 1 : 0), banks = L.n_expert + (L.has_shared ? 1 : 0);
    // Few tokens: the decode kernels. From kGroupedPerBank assignments per bank matrix on average the grouped products
    // (measured: the decode kernels' time grows with the assignments, the grouped products' with the experts they decode, and
    // the two cross at about three assignments per expert), and in any case once the decode kernels no longer read every
    // expert's weights once (they group an expert's rows up to kDecodeDedup assignments a launch).
    // Which grouped products: the descriptor's request (act_blocks), else the faster ones for the formats (int8_faster).
    const bool many = int64_t(n) * slots > std::min<int64_t>(kDecodeDedup, int64_t(kGroupedPerBank) * banks);
    const bool iq4xs = L.gate.type == TQMOE_IQ4_XS && L.down.type == TQMOE_IQ4_XS;
    if (int8_mode_of(L) != 0) p.int8 = int8_ok(L) && (iq4xs ? n >= kGroupedMin : many);
    else p.int8 = int8_ok(L) && many && int8_faster(L.gate.type, n) && int8_faster(L.down.type, n);
    p.grouped = p.int8 || many;
    // the grouped products take 2^24 assignments a pass (32-bit block and byte counts stay far from their limits), the
    // decode kernels 65535
    const int64_t per_pass = p.int8 ? int64_t(1) << 24 : p.grouped ? int64_t(65535 - banks) * 64 : kDecodeAssignments;
    p.chunk = int(std::min<int64_t>(n, std::max<int64_t>(1, per_pass / slots)));
    size_t o = 0;
    auto take = [&](size_t bytes) { const size_t at = o; o = align_up(o + bytes, 256); return at; };
    p.logits = take(size_t(n) * (L.n_expert + 1) * 4);
    p.ids = take(size_t(n) * L.topk * 4);
    p.weights = take(size_t(n) * L.topk * 4);
    p.shared_w = take(size_t(n) * 4);
    p.ids_ext = take(size_t(n) * slots * 4);
    const size_t c = size_t(p.chunk), a = c * slots;
    if (p.grouped) {
        p.counts = take(size_t(banks) * 4);
        p.offsets = take(size_t(banks + 1) * 4);
        p.perm = take(a * 4);
        p.dispatch_ws = take(tqmoe_dispatch_workspace_bytes(banks, p.chunk, slots));
        p.act16 = take(a * L.ff * 2);
        p.y16 = take(a * L.hidden * 4);   // fp16 rows (int8 products) or fp32 rows (fp16 products)
    }
    if (p.int8) {
        const size_t grows = size_t(tqmoe_grouped_rows(int64_t(a), banks));
        p.xq = take(grows * L.hidden);
        const size_t gwords = size_t(tqmoe_grouped_scale_words(int64_t(a), banks));
        p.xs = take(gwords * 4);
        p.aq = take(grows * L.ff);
        p.as = take(gwords * 4);
        p.blocks = act_blocks_of(L) && !plane_gemm_is_fp8(L.gate.type);
        p.rq = take(c * L.hidden);        // the chunk's input rows as int8, quantised once, then gathered per assignment
        p.rs = take(c * 4 * (p.blocks ? size_t(L.hidden / 32) : 1));
        if (p.blocks) {
            p.xbs = take(size_t(tqmoe_grouped_block_scale_words(int64_t(a), banks, L.hidden)) * 4);
            p.abks = take(size_t(tqmoe_grouped_block_scale_words(int64_t(a), banks, L.ff)) * 4);
        }
    } else if (!p.grouped) {
        p.ximage = take(tqmoe_act_image_bytes(n, L.hidden));
        p.aimage = take(tqmoe_act_image_bytes(int32_t(a), L.ff));
        p.y = take(a * L.hidden * 4);
    }
    p.total = o;
    return p;
}

struct Routing { int32_t gating; int32_t norm; const float * bias; };
Routing routing_of(const tqmoe_layer & L) {
    if (L.struct_size < kLayerRoutingSize) return Routing{TQMOE_GATE_SOFTMAX, 1, nullptr};
    return Routing{L.gating ? L.gating : int32_t(TQMOE_GATE_SOFTMAX), L.raw_weights ? 0 : 1, L.probs_bias};
}

int32_t check_layer(const tqmoe_layer * L, tqmoe_error * err) {
    const char * what = "tqmoe_layer_forward";
    if (!L || L->struct_size < kLayerBaseSize) return fail(err, TQMOE_E_ARG, "%s: layer descriptor missing or too small", what);
    const Routing rt = routing_of(*L);
    if (rt.gating < TQMOE_GATE_SOFTMAX || rt.gating > TQMOE_GATE_SQRT_SOFTPLUS) return fail(err, TQMOE_E_UNSUPPORTED, "%s: unsupported gating function %d", what, rt.gating);
    if (L->hidden <= 0 || L->ff <= 0 || L->n_expert <= 0 || L->n_expert > 4096 || L->topk <= 0 || L->topk > L->n_expert || !L->router)
        return fail(err, TQMOE_E_ARG, "%s: invalid layer shape or pointer", what);
    if (L->router_type != TQMOE_F32 && L->router_type != TQMOE_BF16) return fail(err, TQMOE_E_UNSUPPORTED, "%s: router type must be F32 or BF16", what);
    for (const tqmoe_bank * b : {&L->gate, &L->up, &L->down}) if (int32_t rc = check_bank(b, what, err)) return rc;
    const int banks = L->n_expert + (L->has_shared ? 1 : 0);
    if (L->gate.type != L->up.type) return fail(err, TQMOE_E_UNSUPPORTED, "%s: the gate and up banks must share one format (down may have its own)", what);
    if (L->gate.rows != L->ff || L->gate.cols != L->hidden || L->up.rows != L->ff || L->up.cols != L->hidden || L->down.rows != L->hidden ||
        L->down.cols != L->ff || L->gate.experts != banks || L->up.experts != banks || L->down.experts != banks)
        return fail(err, TQMOE_E_ARG, "%s: bank shapes do not match the layer (%d experts of %d x %d expected)", what, banks, L->ff, L->hidden);
    if (L->ff % 32) return fail(err, TQMOE_E_ARG, "%s: ff must be a multiple of 32", what);
    if (L->has_shared && (L->shared_ff <= 0 || L->shared_ff > L->ff || L->shared_ff % 32))
        return fail(err, TQMOE_E_ARG, "%s: shared_ff must be a positive multiple of 32 not above ff", what);
    return 0;
}

}  // namespace
}  // namespace tqmoe

using namespace tqmoe;

extern "C" size_t tqmoe_layer_workspace_bytes(const tqmoe_layer * layer, int32_t n) {
    if (!layer || n <= 0 || check_layer(layer, nullptr)) return 0;
    return plan_for(*layer, n).total;
}

extern "C" int32_t tqmoe_layer_path(const tqmoe_layer * layer, int32_t n) {
    if (!layer || n <= 0 || check_layer(layer, nullptr)) return TQMOE_E_ARG;
    const Plan p = plan_for(*layer, n);
    return p.int8 ? (plane_gemm_is_fp8(layer->gate.type) ? TQMOE_PATH_GROUPED_FP8 : TQMOE_PATH_GROUPED_I8) : p.grouped ? TQMOE_PATH_GROUPED_F16 : TQMOE_PATH_DECODE;
}

static int32_t layer_forward(const tqmoe_layer * layer, const void * x, uint32_t xtype, const void * residual, int32_t n, void * out, uint32_t otype,
                             int32_t * ids_out, float * weights_out, float * logits_out, void * workspace, size_t workspace_bytes, void * stream,
                             tqmoe_error * err) {
    if (int32_t rc = check_layer(layer, err)) return rc;
    const tqmoe_layer & L = *layer;
    if (!x || !out || n <= 0) return fail(err, TQMOE_E_ARG, "tqmoe_layer_forward: invalid shape or pointer");
    if (!is_act_type(xtype) || (otype != TQMOE_F32 && otype != TQMOE_BF16)) return fail(err, TQMOE_E_UNSUPPORTED, "tqmoe_layer_forward: unsupported element type");
    const int slots = L.topk + (L.has_shared ? 1 : 0), banks = L.n_expert + (L.has_shared ? 1 : 0);
    const Plan p = plan_for(L, n);
    if (!workspace || workspace_bytes < p.total) return fail(err, TQMOE_E_WORKSPACE, "tqmoe_layer_forward: workspace of %zu bytes needed", p.total);
    if (int32_t rc = need_device(err, "tqmoe_layer_forward")) return rc;
    uint8_t * ws = static_cast<uint8_t *>(workspace);
    float * logits = logits_out ? logits_out : reinterpret_cast<float *>(ws + p.logits);
    int32_t * ids = ids_out ? ids_out : reinterpret_cast<int32_t *>(ws + p.ids);
    float * weights = weights_out ? weights_out : reinterpret_cast<float *>(ws + p.weights);
    float * shared_w = reinterpret_cast<float *>(ws + p.shared_w);
    const size_t xbytes = elem_bytes(xtype), obytes = elem_bytes(otype);
    const uint8_t * xb = static_cast<const uint8_t *>(x);
    uint8_t * ob = static_cast<uint8_t *>(out);

    if (int32_t rc = tqmoe_router(L.router, L.router_type, L.shared_gate, x, xtype, logits, L.hidden, L.n_expert, n, stream, err)) return rc;
    // one launch: top-k, the ids extended by the shared expert, and (decode path) the input rows' activation image
    int32_t * ext = L.has_shared ? reinterpret_cast<int32_t *>(ws + p.ids_ext) : nullptr;
    const Routing rt = routing_of(L);
    const Glu glu = glu_of(L);
    enqueue_topk(logits, ids, weights, shared_w, ext, L.n_expert, x, xtype, L.hidden, p.grouped ? nullptr : ws + p.ximage, L.n_expert, L.topk, n,
                 L.weight_scale, rt.gating, rt.bias, rt.norm, static_cast<hipStream_t>(stream), L.has_shared && !L.shared_gate);
    if (int32_t rc = launched(err, "tqmoe_layer_forward (top-k)")) return rc;
    const int32_t * ids_ext = ext ? ext : ids;

    for (int t0 = 0; t0 < n; t0 += p.chunk) {
        const int c = std::min(p.chunk, n - t0);
        const int32_t * cid = ids_ext + size_t(t0) * slots;
        const float * cw = weights + size_t(t0) * L.topk, * csw = shared_w + t0;
        void * cout = ob + size_t(t0) * L.hidden * obytes;
        // the weighted sum of the chunk's rows, with the residual rows added when the caller gave them
        auto combine = [&](const void * routed, uint32_t rtype, const void * shared) -> int32_t {
            if (residual)
                return tqmoe_combine_residual(routed, rtype, slots, shared, int64_t(slots) * L.hidden, cw, csw,
                                              static_cast<const uint8_t *>(residual) + size_t(t0) * L.hidden * 2, cout, L.hidden, L.topk, c, stream, err);
            if (rtype == TQMOE_F16)
                return tqmoe_combine_strided_f16(routed, slots, shared, int64_t(slots) * L.hidden, cw, csw, cout, otype, L.hidden, L.topk, c, stream, err);
            return tqmoe_combine_strided(static_cast<const float *>(routed), slots, static_cast<const float *>(shared), int64_t(slots) * L.hidden, cw, csw, cout, otype,
                                         L.hidden, L.topk, c, stream, err);
        };
        if (p.grouped) {
            int8_t * xq = reinterpret_cast<int8_t *>(ws + p.xq), * aq = reinterpret_cast<int8_t *>(ws + p.aq);
            float * xs = reinterpret_cast<float *>(ws + p.xs), * as = reinterpret_cast<float *>(ws + p.as);
            int32_t * counts = reinterpret_cast<int32_t *>(ws + p.counts), * offsets = reinterpret_cast<int32_t *>(ws + p.offsets),
                    * perm = reinterpret_cast<int32_t *>(ws + p.perm);
            uint16_t * act16 = reinterpret_cast<uint16_t *>(ws + p.act16), * y16 = reinterpret_cast<uint16_t *>(ws + p.y16);
            if (int32_t rc = tqmoe_dispatch(cid, counts, offsets, perm, nullptr, 0, banks, c, slots, ws + p.dispatch_ws,
                                            tqmoe_dispatch_workspace_bytes(banks, c, slots), stream, err)) return rc;
            if (!p.int8) {
                if (int32_t rc = gemm_f16_common(&L.gate, &L.up, xb + size_t(t0) * L.hidden * xbytes, xtype, counts, offsets, perm, c, slots, L.topk, L.shared_ff, slots,
                                                 act16, TQMOE_F16, 1, stream, err, "tqmoe_layer_forward (gate / up)", glu)) return rc;
                float * y32 = reinterpret_cast<float *>(y16);
                if (int32_t rc = tqmoe_expert_gemm(&L.down, act16, TQMOE_F16, counts, offsets, perm, c, slots, L.topk, L.shared_ff, 1, y32, TQMOE_F32, stream, err)) return rc;
                if (int32_t rc = combine(y32, TQMOE_F32, L.has_shared ? y32 + size_t(L.topk) * L.hidden : nullptr)) return rc;
                continue;
            } else {
            int8_t * rq = reinterpret_cast<int8_t *>(ws + p.rq);
            float * rs = reinterpret_cast<float *>(ws + p.rs);
            if (plane_gemm_is_fp8(L.gate.type)) {
                if (int32_t rc = tqmoe_quant_rows_fp8(xb + size_t(t0) * L.hidden * xbytes, xtype, c, L.hidden, reinterpret_cast<uint8_t *>(rq), rs, stream, err)) return rc;
                if (int32_t rc = tqmoe_gather_rows_i8(rq, rs, L.hidden, counts, offsets, perm, banks, int64_t(c) * slots, slots, xq, xs, stream, err)) return rc;
                if (int32_t rc = gemm_8bit_common(&L.gate, &L.up, xq, xs, counts, offsets, perm, c, slots, L.topk, L.shared_ff, act16, 1, stream, err,
                                                  "tqmoe_layer_forward (gate / up)", true, nullptr, false, glu, 0, nullptr)) return rc;
                if (int32_t rc = group_rows_common(act16, TQMOE_F16, L.ff, counts, offsets, perm, banks, int64_t(c) * slots, 1, aq, as, stream, err, true,
                                                   "tqmoe_layer_forward (act rows)", nullptr, false, xs)) return rc;
                if (int32_t rc = gemm_8bit_common(&L.down, nullptr, aq, as, counts, offsets, perm, c, slots, L.topk, L.shared_ff, y16, 0, stream, err,
                                                  "tqmoe_layer_forward (down)", true, nullptr, false, Glu{0.f, 0}, 0, xs)) return rc;
            } else if (p.blocks) {
            float * xbs = reinterpret_cast<float *>(ws + p.xbs), * abks = reinterpret_cast<float *>(ws + p.abks);
            if (int32_t rc = tqmoe_quant_rows_i8_blocks(xb + size_t(t0) * L.hidden * xbytes, xtype, c, L.hidden, rq, rs, nullptr, stream, err)) return rc;
            if (int32_t rc = tqmoe_gather_rows_i8_blocks(rq, rs, L.hidden, counts, offsets, perm, banks, int64_t(c) * slots, slots, xq, xs, xbs, stream, err)) return rc;
            if (int32_t rc = gemm_8bit_common(&L.gate, &L.up, xq, xs, counts, offsets, perm, c, slots, L.topk, L.shared_ff, act16, 1, stream, err,
                                              "tqmoe_layer_forward (gate / up)", false, xbs, true, glu, 0, nullptr)) return rc;
            if (int32_t rc = group_rows_common(act16, TQMOE_F16, L.ff, counts, offsets, perm, banks, int64_t(c) * slots, 1, aq, as, stream, err, false,
                                               "tqmoe_layer_forward (act rows)", abks, true, xs)) return rc;
            if (int32_t rc = gemm_8bit_common(&L.down, nullptr, aq, as, counts, offsets, perm, c, slots, L.topk, L.shared_ff, y16, 0, stream, err,
                                              "tqmoe_layer_forward (down)", false, abks, true, Glu{0.f, 0}, 0, xs)) return rc;
            } else {
            if (int32_t rc = tqmoe_quant_rows_i8(xb + size_t(t0) * L.hidden * xbytes, xtype, c, L.hidden, rq, rs, stream, err)) return rc;
            if (int32_t rc = tqmoe_gather_rows_i8(rq, rs, L.hidden, counts, offsets, perm, banks, int64_t(c) * slots, slots, xq, xs, stream, err)) return rc;
            if (int32_t rc = gemm_8bit_common(&L.gate, &L.up, xq, xs, counts, offsets, perm, c, slots, L.topk, L.shared_ff, act16, 1, stream, err,
                                              "tqmoe_layer_forward (gate / up)", false, nullptr, false, glu, 0, nullptr)) return rc;
            if (int32_t rc = group_rows_common(act16, TQMOE_F16, L.ff, counts, offsets, perm, banks, int64_t(c) * slots, 1, aq, as, stream, err, false,
                                               "tqmoe_layer_forward (act rows)", nullptr, false, xs)) return rc;
            if (int32_t rc = gemm_8bit_common(&L.down, nullptr, aq, as, counts, offsets, perm, c, slots, L.topk, L.shared_ff, y16, 0, stream, err,
                                              "tqmoe_layer_forward (down)", false, nullptr, false, Glu{0.f, 0}, 0, xs)) return rc;
            }
            }
            if (int32_t rc = combine(y16, TQMOE_F16, L.has_shared ? y16 + size_t(L.topk) * L.hidden : nullptr)) return rc;
        } else {
            const uint8_t * ximage = ws + p.ximage + tqmoe_act_image_bytes(1, L.hidden) * size_t(t0);
            float * y = reinterpret_cast<float *>(ws + p.y);
            if (int32_t rc = expert_gateup_glu(&L.gate, &L.up, ximage, ws + p.aimage, cid, c, slots, L.topk, L.shared_ff, glu, stream, err)) return rc;
            if (int32_t rc = tqmoe_expert_down(&L.down, ws + p.aimage, y, cid, c, slots, L.topk, L.shared_ff, stream, err)) return rc;
            if (int32_t rc = combine(y, TQMOE_F32, L.has_shared ? y + size_t(L.topk) * L.hidden : nullptr)) return rc;
        }
    }
    return ok(err);
}

extern "C" int32_t tqmoe_layer_forward(const tqmoe_layer * layer, const void * x, uint32_t xtype, int32_t n, void * out, uint32_t otype,
                                       int32_t * ids_out, float * weights_out, float * logits_out, void * workspace, size_t workspace_bytes,
                                       void * stream, tqmoe_error * err) {
    return layer_forward(layer, x, xtype, nullptr, n, out, otype, ids_out, weights_out, logits_out, workspace, workspace_bytes, stream, err);
}

extern "C" int32_t tqmoe_layer_forward_residual(const tqmoe_layer * layer, const void * x, uint32_t xtype, const void * residual, int32_t n, void * out,
                                                int32_t * ids_out, float * weights_out, float * logits_out, void * workspace, size_t workspace_bytes,
                                                void * stream, tqmoe_error * err) {
    if (!residual) return fail(err, TQMOE_E_ARG, "tqmoe_layer_forward_residual: residual rows missing");
    return layer_forward(layer, x, xtype, residual, n, out, TQMOE_BF16, ids_out, weights_out, logits_out, workspace, workspace_bytes, stream, err);
}

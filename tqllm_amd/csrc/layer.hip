// The whole layer behind one entry point: router -> top-k -> activation image -> gate/up + SwiGLU -> down + combine.
#include "formats.cuh"

namespace tqmoe {
int32_t check_bank(const tqmoe_bank * b, const char * what, tqmoe_error * err);
int32_t enqueue_topk(const float * logits, int32_t * ids, float * weights, float * shared_weights, int32_t * ext_ids, int32_t extra, const void * x,
                     uint32_t xtype, int32_t cols, void * image, int32_t experts, int32_t topk, int32_t n, float scale, hipStream_t s);

namespace {

struct Plan {  // byte offsets into the workspace
    size_t logits, ids, weights, shared_w, ids_ext, ximage, aimage, y, total;
};

Plan plan_for(const tqmoe_layer & L, int n) {
    Plan p{};
    const int slots = L.topk + (L.has_shared ? 1 : 0);
    size_t o = 0;
    auto take = [&](size_t bytes) { const size_t at = o; o = align_up(o + bytes, 256); return at; };
    p.logits = take(size_t(n) * (L.n_expert + 1) * 4);
    p.ids = take(size_t(n) * L.topk * 4);
    p.weights = take(size_t(n) * L.topk * 4);
    p.shared_w = take(size_t(n) * 4);
    p.ids_ext = take(size_t(n) * slots * 4);
    p.ximage = take(tqmoe_act_image_bytes(n, L.hidden));
    p.aimage = take(tqmoe_act_image_bytes(n * slots, L.ff));
    p.y = take(size_t(n) * slots * L.hidden * 4);
    p.total = o;
    return p;
}

int32_t check_layer(const tqmoe_layer * L, tqmoe_error * err) {
    const char * what = "tqmoe_layer_forward";
    if (!L || L->struct_size < sizeof(tqmoe_layer)) return fail(err, TQMOE_E_ARG, "%s: layer descriptor missing or too small", what);
    if (L->hidden <= 0 || L->ff <= 0 || L->n_expert <= 0 || L->n_expert > 4096 || L->topk <= 0 || L->topk > L->n_expert || !L->router)
        return fail(err, TQMOE_E_ARG, "%s: invalid layer shape or pointer", what);
    if (L->router_type != TQMOE_F32 && L->router_type != TQMOE_BF16) return fail(err, TQMOE_E_UNSUPPORTED, "%s: router type must be F32 or BF16", what);
    for (const tqmoe_bank * b : {&L->gate, &L->up, &L->down}) if (int32_t rc = check_bank(b, what, err)) return rc;
    const int banks = L->n_expert + (L->has_shared ? 1 : 0);
    if (L->gate.type != L->up.type || L->gate.type != L->down.type) return fail(err, TQMOE_E_UNSUPPORTED, "%s: the three banks must share one format", what);
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

extern "C" int32_t tqmoe_layer_forward(const tqmoe_layer * layer, const void * x, uint32_t xtype, int32_t n, void * out, uint32_t otype,
                                       int32_t * ids_out, float * weights_out, float * logits_out, void * workspace, size_t workspace_bytes,
                                       void * stream, tqmoe_error * err) {
    if (int32_t rc = check_layer(layer, err)) return rc;
    const tqmoe_layer & L = *layer;
    if (!x || !out || n <= 0) return fail(err, TQMOE_E_ARG, "tqmoe_layer_forward: invalid shape or pointer");
    if (!is_act_type(xtype) || (otype != TQMOE_F32 && otype != TQMOE_BF16)) return fail(err, TQMOE_E_UNSUPPORTED, "tqmoe_layer_forward: unsupported element type");
    const int slots = L.topk + (L.has_shared ? 1 : 0);
    if (int64_t(n) * slots > 65535) return fail(err, TQMOE_E_UNSUPPORTED, "tqmoe_layer_forward: n * (topk + shared) exceeds 65535 on the decode path");
    const Plan p = plan_for(L, n);
    if (!workspace || workspace_bytes < p.total) return fail(err, TQMOE_E_WORKSPACE, "tqmoe_layer_forward: workspace of %zu bytes needed", p.total);
    if (int32_t rc = need_device(err, "tqmoe_layer_forward")) return rc;
    uint8_t * ws = static_cast<uint8_t *>(workspace);
    float * logits = logits_out ? logits_out : reinterpret_cast<float *>(ws + p.logits);
    int32_t * ids = ids_out ? ids_out : reinterpret_cast<int32_t *>(ws + p.ids);
    float * weights = weights_out ? weights_out : reinterpret_cast<float *>(ws + p.weights);
    float * shared_w = reinterpret_cast<float *>(ws + p.shared_w);

    if (int32_t rc = tqmoe_router(L.router, L.router_type, L.shared_gate, x, xtype, logits, L.hidden, L.n_expert, n, stream, err)) return rc;
    // one launch: softmax top-k, the ids extended by the shared expert, and the input rows' activation image
    int32_t * ext = L.has_shared ? reinterpret_cast<int32_t *>(ws + p.ids_ext) : nullptr;
    enqueue_topk(logits, ids, weights, shared_w, ext, L.n_expert, x, xtype, L.hidden, ws + p.ximage, L.n_expert, L.topk, n, L.weight_scale,
                 static_cast<hipStream_t>(stream));
    if (int32_t rc = launched(err, "tqmoe_layer_forward (top-k)")) return rc;
    const int32_t * ids_ext = ext ? ext : ids;
    float * y = reinterpret_cast<float *>(ws + p.y);
    if (int32_t rc = tqmoe_expert_gateup(&L.gate, &L.up, ws + p.ximage, ws + p.aimage, ids_ext, n, slots, L.topk, L.shared_ff, stream, err)) return rc;
    if (int32_t rc = tqmoe_expert_down(&L.down, ws + p.aimage, y, ids_ext, n, slots, L.topk, L.shared_ff, stream, err)) return rc;
    return tqmoe_combine_strided(y, slots, L.has_shared ? y + size_t(L.topk) * L.hidden : nullptr, int64_t(slots) * L.hidden, weights, shared_w, out, otype,
                                 L.hidden, L.topk, n, stream, err);
}

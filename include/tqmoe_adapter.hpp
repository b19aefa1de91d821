// C++ face of the tqmoe C ABI with the names and error behaviour of the reference's own interfaces, header-only.
//
//   namespace tqmoe_hip   the free functions of `namespace tqllm_cuda` (src/experts/moe_kernels.cuh:7-81): same names,
//                         same argument order and meaning; streams are `void *` (a hipStream_t); bad shapes throw
//                         std::invalid_argument and device failures std::runtime_error, as moe.cu:239, 250-251, 269 do.
//   tqmoe_hip::ExpertFormat   the expert entry points of `tqllm::WeightFormat` (weight_format.hpp:51-73) over a bank
//                         view: a `bool false` return means "this format has no such kernel, fall back", as there.
//
// Differences a caller has to know, all of them in the element types (the reference's kernels speak fp16 / bf16; this
// library takes the element type as an argument and keeps intermediate rows in fp32 or in its private activation image):
// they are spelled out at each function.
#pragma once
#include <stdexcept>
#include <string>

#include "tqmoe.h"

namespace tqmoe_hip {

inline void check(int32_t rc, const tqmoe_error & e) {
    if (rc == TQMOE_OK) return;
    const std::string msg = e.message[0] ? e.message : "tqmoe call failed";
    if (rc == TQMOE_E_ARG || rc == TQMOE_E_UNSUPPORTED || rc == TQMOE_E_WORKSPACE) throw std::invalid_argument(msg);
    throw std::runtime_error(msg);
}
inline tqmoe_error fresh() {
    tqmoe_error e{};
    e.struct_size = sizeof(tqmoe_error);
    return e;
}

// moe_router / moe_router_f32 (moe_kernels.cuh:7-10): fp32 router rows; x fp16 or fp32. moe_router_bf16 is the Flash-Next
// form (bf16 router rows, bf16 x; qwen4exp.cu:1629-1659).
inline void moe_router(const float * router, const float * shared_gate, const void * x_f16, float * logits, int hidden, int experts, int n, void * stream) {
    tqmoe_error e = fresh();
    check(tqmoe_router(router, TQMOE_F32, shared_gate, x_f16, TQMOE_F16, logits, hidden, experts, n, stream, &e), e);
}
inline void moe_router_f32(const float * router, const float * shared_gate, const float * x, float * logits, int hidden, int experts, int n, void * stream) {
    tqmoe_error e = fresh();
    check(tqmoe_router(router, TQMOE_F32, shared_gate, x, TQMOE_F32, logits, hidden, experts, n, stream, &e), e);
}
inline void moe_router_bf16(const void * router_bf16, const void * shared_gate_bf16, const void * x_bf16, float * logits, int hidden, int experts, int n,
                            void * stream) {
    tqmoe_error e = fresh();
    check(tqmoe_router(router_bf16, TQMOE_BF16, shared_gate_bf16, x_bf16, TQMOE_BF16, logits, hidden, experts, n, stream, &e), e);
}
// moe_topk (moe_kernels.cuh:19-20)
inline void moe_topk(const float * logits, int * ids, float * weights, float * shared_weights, int experts, int topk, int n, float scale, void * stream) {
    tqmoe_error e = fresh();
    check(tqmoe_topk(logits, ids, weights, shared_weights, experts, topk, n, scale, stream, &e), e);
}
// moe_topk2 (moe_kernels.cuh:24-25): two routings in one launch
inline void moe_topk2(const float * logits, int * ids, float * weights, float * shared_weights, const float * logits2, int * ids2, float * weights2,
                      float * shared_weights2, int e, int k, int n, float scale, void * stream) {
    tqmoe_error err = fresh();
    check(tqmoe_topk2(logits, ids, weights, shared_weights, logits2, ids2, weights2, shared_weights2, e, k, n, scale, stream, &err), err);
}
// moe_route (src/experts/moe.hpp:28-51) for n tokens on the device: the host function's configuration with its defaults
// (sigmoid gating, weights not normalised, no scale); logits rows hold n_expert + 1 columns as moe_router writes them,
// probs_bias is a device array of n_expert floats or null. Throws for a gating value outside MoeGating's.
struct MoeRouting {
    int n_expert = 0;
    int n_expert_used = 0;
    int gating = TQMOE_GATE_SIGMOID;
    bool norm_weights = false;
    float weight_scale = 0.f;
};
inline void moe_route(const MoeRouting & cfg, const float * logits, const float * probs_bias, int * ids, float * weights, float * shared_weights, int n,
                      void * stream) {
    tqmoe_error e = fresh();
    check(tqmoe_topk_gated(logits, probs_bias, cfg.gating, cfg.norm_weights ? 1 : 0, ids, weights, shared_weights, cfg.n_expert, cfg.n_expert_used, n,
                           cfg.weight_scale, stream, &e), e);
}
// The step in front of the layer, the pair add_sumsq + norm_h of Qwen35Engine::ffn_block (qwen35_forward.cpp:1114-1115) in
// one launch: m += residual (bf16, in place; residual may be null), xh = fp16(bf16(m * inv * w)). No partial-sum buffer.
inline void add_norm_h(void * m_bf16, const void * residual_bf16, const float * w, float eps, void * xh_f16, int hidden, int n, void * stream) {
    tqmoe_error e = fresh();
    check(tqmoe_add_rmsnorm(m_bf16, residual_bf16, w, eps, xh_f16, TQMOE_F16, hidden, n, stream, &e), e);
}
// moe_sum followed by the residual add (qwen35_forward.cpp:1248-1250): x = bf16(bf16(sum) + m); x may be m's buffer
inline void moe_sum_add(const float * routed, const float * shared, const float * weights, const float * shared_weights, const void * m_bf16, void * x_bf16,
                        int hidden, int topk, int n, void * stream) {
    tqmoe_error e = fresh();
    check(tqmoe_combine_residual(routed, TQMOE_F32, topk, shared, hidden, weights, shared_weights, m_bf16, x_bf16, hidden, topk, n, stream, &e), e);
}
// moe_group (moe_kernels.cuh:29), the reference's signature: groups [experts][n], counts [experts]; negative ids are skipped.
// The lists are ascending inside each expert (the reference's device version is atomic-ordered). No workspace: the chunk
// counts live in the library's own device image (tqmoe_dispatch_static), so calls that overlap in time on one GPU must not
// be issued from two streams.
inline void moe_group(const int * ids, int * counts, int * groups, int experts, int n, int topk, void * stream) {
    tqmoe_error e = fresh();
    check(tqmoe_dispatch_static(ids, counts, nullptr, nullptr, groups, n, experts, n, topk, stream, &e), e);
}
// moe_count (moe_kernels.cuh, moe.cu:183-186): counts[ids[i]] += 1, 64-bit counters
inline void moe_count(const int * ids, unsigned long long * counts, int count, void * stream) {
    tqmoe_error e = fresh();
    check(tqmoe_count(ids, reinterpret_cast<uint64_t *>(counts), count, stream, &e), e);
}
// moe_dedup_maps (moe_kernels.cuh:34-39) with the map layout of quant_kernels.cuh:26-27
constexpr int kDedupCols = 8, kDedupStride = 2 + 2 * kDedupCols;
inline void moe_dedup_maps(const int * ids, const int * slot_of, int count, int topk, int * slots, int * gu, int * dn, int groups, void * stream) {
    tqmoe_error e = fresh();
    check(tqmoe_dedup_maps(ids, slot_of, count, topk, slots, gu, dn, groups, stream, &e), e);
}
// moe_swiglu (moe_kernels.cuh:71-72), fp32 in and out here; swiglu_clamp / clamp_gate: MoeConfig::swiglu_clamp and the switch
// of moe_expert_ffn (src/experts/moe.hpp:34-36, moe.cpp:128-143), off by default
inline void moe_swiglu(const float * gate, const float * up, float * act, int count, void * stream, float swiglu_clamp = 0.f, bool clamp_gate = false) {
    tqmoe_error e = fresh();
    check(tqmoe_swiglu_clamped(gate, up, act, count, swiglu_clamp, clamp_gate ? 1 : 0, stream, &e), e);
}
// moe_sum (moe_kernels.cuh:73-74): routed / shared fp32 here, out bf16 as there
inline void moe_sum(const float * routed, const float * shared, const float * weights, const float * shared_weights, void * out_bf16, int hidden, int topk, int n,
                    void * stream) {
    tqmoe_error e = fresh();
    check(tqmoe_combine(routed, shared, weights, shared_weights, out_bf16, TQMOE_BF16, hidden, topk, n, stream, &e), e);
}
// moe_extend_ids (moe_kernels.cuh:77-78) without the hot / cold slot maps
inline void moe_extend_ids(const int * ids, int * out, int k, int n, int extra, void * stream) {
    tqmoe_error e = fresh();
    check(tqmoe_extend_ids(ids, out, k, n, extra, stream, &e), e);
}
// moe_sum_strided (moe_kernels.cuh:80-81)
inline void moe_sum_strided(const float * routed, int slots, const float * shared, int shared_ld, const float * weights, const float * shared_weights,
                            void * out_bf16, int hidden, int topk, int n, void * stream) {
    tqmoe_error e = fresh();
    check(tqmoe_combine_strided(routed, slots, shared, shared_ld, weights, shared_weights, out_bf16, TQMOE_BF16, hidden, topk, n, stream, &e), e);
}

// The expert entry points of tqllm::WeightFormat over a bank view (the Mat of stacked experts, weight_format.hpp:22-28, 61).
struct ExpertFormat {
    // WeightFormat::load (weight_format.hpp:41): raw GGUF bytes already on the device -> the two planes (caller memory of
    // tqmoe_bank_layout's sizes). Throws like the loaders do on a rejected row (q4.cpp:519-521) when `status` is read back
    // by the caller; here only argument errors throw.
    static tqmoe_bank load(uint32_t type, const void * gguf_blocks_dev, int experts, int rows, int cols, void * codes, void * aux, int32_t * status_dev, void * stream) {
        tqmoe_error e = fresh();
        check(tqmoe_bank_load(type, gguf_blocks_dev, int64_t(experts) * rows, cols, codes, aux, status_dev, stream, &e), e);
        tqmoe_bank b{};
        b.struct_size = sizeof(tqmoe_bank);
        b.type = type; b.experts = experts; b.rows = rows; b.cols = cols; b.codes = codes; b.aux = aux;
        return b;
    }
    static bool has_expert_matvec() { return true; }
    // expert_matvec (weight_format.hpp:62-64): x arrives as the activation image of the input rows (tqmoe_quant_act);
    // y [n * topk][rows] of ytype (TQMOE_BF16 gives the reference's output type).
    static void expert_matvec(const tqmoe_bank & m, const void * x_image, void * y, uint32_t ytype, const int * ids, int n, int topk, bool per_expert_input,
                              void * stream) {
        tqmoe_error e = fresh();
        check(tqmoe_expert_matvec(&m, x_image, y, ytype, ids, n, topk, per_expert_input ? 1 : 0, stream, &e), e);
    }
    // expert_matvec2 (weight_format.hpp:70-73)
    static void expert_matvec2(const tqmoe_bank & g, const tqmoe_bank & u, const void * x_image, void * yg, void * yu, uint32_t ytype, const int * ids, int n,
                               int topk, void * stream) {
        tqmoe_error e = fresh();
        check(tqmoe_expert_matvec2(&g, &u, x_image, yg, yu, ytype, ids, n, topk, stream, &e), e);
    }
    // expert_gemm_i8 (weight_format.hpp:54-56), mode 2 (one scale per token row), lists as counts / offsets / perm;
    // false: no grouped int8 kernel for this format.
    static bool expert_gemm_i8(const tqmoe_bank & m, const int8_t * xq, const float * xs, void * y_f16, const int * counts, const int * offsets, const int * perm,
                               int n, int topk, void * stream) {
        tqmoe_error e = fresh();
        const int32_t rc = tqmoe_expert_gemm_i8(&m, xq, xs, counts, offsets, perm, n, topk, topk, 0, y_f16, stream, &e);
        if (rc == TQMOE_E_UNSUPPORTED) return false;
        check(rc, e);
        return true;
    }
    // expert_gemm_gateup (weight_format.hpp:57-59) on int8 rows; y [assignments][rows] half
    static bool expert_gemm_gateup_i8(const tqmoe_bank & g, const tqmoe_bank & u, const int8_t * xq, const float * xs, void * y_f16, const int * counts,
                                   const int * offsets, const int * perm, int n, int topk, void * stream) {
        tqmoe_error e = fresh();
        const int32_t rc = tqmoe_expert_gemm_gateup_i8(&g, &u, xq, xs, counts, offsets, perm, n, topk, topk, 0, y_f16, stream, &e);
        if (rc == TQMOE_E_UNSUPPORTED) return false;
        check(rc, e);
        return true;
    }
    // the two int8 products in mode 1 (a scale per 32 values of every row, quant_kernels.cuh:13-16): block_scale is
    // tqmoe_group_rows_i8_blocks' third output for the same lists
    static bool expert_gemm_i8_blocks(const tqmoe_bank & m, const int8_t * xq, const float * xs, const float * block_scale, void * y_f16, const int * counts,
                                      const int * offsets, const int * perm, int n, int topk, void * stream) {
        tqmoe_error e = fresh();
        const int32_t rc = tqmoe_expert_gemm_i8_blocks(&m, xq, xs, block_scale, counts, offsets, perm, n, topk, topk, 0, y_f16, stream, &e);
        if (rc == TQMOE_E_UNSUPPORTED) return false;
        check(rc, e);
        return true;
    }
    static bool expert_gemm_gateup_i8_blocks(const tqmoe_bank & g, const tqmoe_bank & u, const int8_t * xq, const float * xs, const float * block_scale, void * y_f16,
                                             const int * counts, const int * offsets, const int * perm, int n, int topk, void * stream) {
        tqmoe_error e = fresh();
        const int32_t rc = tqmoe_expert_gemm_gateup_i8_blocks(&g, &u, xq, xs, block_scale, counts, offsets, perm, n, topk, topk, 0, y_f16, stream, &e);
        if (rc == TQMOE_E_UNSUPPORTED) return false;
        check(rc, e);
        return true;
    }
    // the same two products on E4M3 rows for NVFP4G banks (rows of tqmoe_group_rows_fp8, scale amax / 448 as
    // src/core/fp8_gemm.cuh:19-31); false: the format has no fp8 grouped kernel
    static bool expert_gemm_fp8(const tqmoe_bank & m, const uint8_t * xq, const float * xs, void * y_f16, const int * counts, const int * offsets, const int * perm,
                                int n, int topk, void * stream) {
        tqmoe_error e = fresh();
        const int32_t rc = tqmoe_expert_gemm_fp8(&m, xq, xs, counts, offsets, perm, n, topk, topk, 0, y_f16, stream, &e);
        if (rc == TQMOE_E_UNSUPPORTED) return false;
        check(rc, e);
        return true;
    }
    static bool expert_gemm_gateup_fp8(const tqmoe_bank & g, const tqmoe_bank & u, const uint8_t * xq, const float * xs, void * y_f16, const int * counts,
                                       const int * offsets, const int * perm, int n, int topk, void * stream) {
        tqmoe_error e = fresh();
        const int32_t rc = tqmoe_expert_gemm_gateup_fp8(&g, &u, xq, xs, counts, offsets, perm, n, topk, topk, 0, y_f16, stream, &e);
        if (rc == TQMOE_E_UNSUPPORTED) return false;
        check(rc, e);
        return true;
    }
    // expert_gemm (weight_format.hpp:51-53) for any bank format: half input rows [n][cols] (or one row per assignment with
    // per_expert_input), y [n * topk][rows] half. Weights are decoded to fp16 tiles on the fly; fp32 accumulation.
    static bool expert_gemm(const tqmoe_bank & m, const void * x_f16, void * y_f16, const int * counts, const int * offsets, const int * perm, int n, int topk,
                            bool per_expert_input, void * stream) {
        tqmoe_error e = fresh();
        const int32_t rc = tqmoe_expert_gemm(&m, x_f16, TQMOE_F16, counts, offsets, perm, n, topk, topk, 0, per_expert_input ? 1 : 0, y_f16, TQMOE_F16, stream, &e);
        if (rc == TQMOE_E_UNSUPPORTED) return false;
        check(rc, e);
        return true;
    }
    // expert_gemm_gateup (weight_format.hpp:57-59) for any bank format on half input rows; act [n * topk][rows] half
    static bool expert_gemm_gateup(const tqmoe_bank & g, const tqmoe_bank & u, const void * x_f16, void * act_f16, const int * counts, const int * offsets,
                                   const int * perm, int n, int topk, void * stream) {
        tqmoe_error e = fresh();
        const int32_t rc = tqmoe_expert_gemm_gateup(&g, &u, x_f16, TQMOE_F16, counts, offsets, perm, n, topk, topk, 0, act_f16, stream, &e);
        if (rc == TQMOE_E_UNSUPPORTED) return false;
        check(rc, e);
        return true;
    }
    // dequant_rows_h (weight_format.hpp:84-86) with fp32 output: the decoded values bit for bit
    static bool dequant_rows(const tqmoe_bank & m, float * out, int64_t row0, int64_t nrows, void * stream) {
        tqmoe_error e = fresh();
        check(tqmoe_bank_dequant(&m, row0, nrows, out, stream, &e), e);
        return true;
    }
};

// The expert virtuals of tqllm::WeightFormat with the base class's exact signatures (weight_format.hpp:51-73), as a mixin
// over the reference's own types, so that a maintainer derives the HIP format from it and the `override`s compile:
//
//   struct HipExperts final : tqmoe_hip::ExpertOverrides<tqllm::WeightFormat, tqllm::Mat, __half, __nv_bfloat16, cudaStream_t> { ... };
//
// Mat is read as the reference fills it for stacked experts (weight_format.hpp:22-28, 61): p = code plane, aux = aux
// plane, type = GGUF type id, rows = experts * rows of one expert, cols. The base signatures carry no scratch memory and
// no token count, so the object holds them: `scratch` is engine-owned device memory (set_scratch) for the activation
// image of a decode call and for the offsets / permutation form of a grouped call's lists
// (expert_scratch_bytes(rows, cols, assignments, experts) bytes); `max_assignments` bounds the listed assignments of a
// grouped call (n * topk of the pass; 0 = experts * capacity, always safe, costs idle blocks). Return values and
// exceptions are the base's: false = "no such kernel for this format, fall back", std::invalid_argument on bad shapes,
// std::runtime_error on device errors.
// int8_mode: 0 = no expert_gemm_i8 calls, else the largest mode they will pass (1 needs room for the block scales too)
inline size_t expert_scratch_bytes(int cols, int input_rows, int max_assignments, int experts, int int8_mode = 0) {
    const size_t image = tqmoe_act_image_bytes(input_rows, cols);
    const size_t lists = (2 * size_t(experts) + 1 + size_t(max_assignments)) * 4 + 1024;
    const size_t i8 = int8_mode ? tqmoe_expert_gemm_i8_ref_scratch_bytes(experts, max_assignments, cols, int8_mode == 1 ? 1 : 2) : 0;
    return image > lists ? (image > i8 ? image : i8) : (lists > i8 ? lists : i8);
}

template <class Base, class MatT, class HalfT, class Bf16T, class StreamT>
struct ExpertOverrides : Base {
    void * scratch = nullptr;
    size_t scratch_bytes = 0;
    int max_assignments = 0;
    void set_scratch(void * device_memory, size_t bytes) { scratch = device_memory; scratch_bytes = bytes; }

    static tqmoe_bank bank_of(const MatT & m, int rows) {
        tqmoe_bank b{};
        b.struct_size = sizeof(tqmoe_bank);
        b.type = m.type; b.experts = rows > 0 ? m.rows / rows : 0; b.rows = rows; b.cols = m.cols; b.codes = m.p; b.aux = m.aux;
        return b;
    }
    bool has_expert_matvec() const override { return true; }

    void expert_matvec(const MatT & m, const HalfT * x, Bf16T * y, int rows, const int * ids, int n, int topk, bool per_expert_input, StreamT stream) const override {
        tqmoe_error e = fresh();
        const tqmoe_bank b = bank_of(m, rows);
        check(tqmoe_expert_matvec_rows(&b, x, TQMOE_F16, y, TQMOE_BF16, ids, n, topk, per_expert_input ? 1 : 0, scratch, scratch_bytes, (void *)stream, &e), e);
    }
    void expert_matvec2(const MatT & g, const MatT & u, const HalfT * x, Bf16T * yg, Bf16T * yu, int rows, const int * ids, int n, int topk,
                        StreamT stream) const override {
        tqmoe_error e = fresh();
        const tqmoe_bank bg = bank_of(g, rows), bu = bank_of(u, rows);
        check(tqmoe_expert_matvec2_rows(&bg, &bu, x, TQMOE_F16, yg, yu, TQMOE_BF16, ids, n, topk, scratch, scratch_bytes, (void *)stream, &e), e);
    }
    // expert_matvec_dedup / expert_matvec_dedup2 (weight_format.hpp:66-69) over the maps of moe_dedup_maps; the scratch must hold
    // tqmoe_expert_matvec_dedup_scratch_bytes(groups, rows, cols, TQMOE_BF16, two banks). The base's has_expert_dedup() follows its
    // u4h_id(), which stays -1 here (the id selects kernels of the reference's own u4h family): an engine that asks
    // has_expert_dedup() finds these, one that asks u4h_id() takes expert_matvec, which serves an expert's rows together as well.
    bool has_expert_dedup() const override { return true; }
    void expert_matvec_dedup(const MatT & m, const HalfT * x, Bf16T * y, int rows, const int * dmap, int groups, StreamT stream) const override {
        tqmoe_error e = fresh();
        const tqmoe_bank b = bank_of(m, rows);
        check(tqmoe_expert_matvec_dedup(&b, nullptr, x, TQMOE_F16, y, nullptr, TQMOE_BF16, dmap, groups, scratch, scratch_bytes, (void *)stream, &e), e);
    }
    void expert_matvec_dedup2(const MatT & g, const MatT & u, const HalfT * x, Bf16T * yg, Bf16T * yu, int rows, const int * dmap, int groups,
                              StreamT stream) const override {
        tqmoe_error e = fresh();
        const tqmoe_bank bg = bank_of(g, rows), bu = bank_of(u, rows);
        check(tqmoe_expert_matvec_dedup(&bg, &bu, x, TQMOE_F16, yg, yu, TQMOE_BF16, dmap, groups, scratch, scratch_bytes, (void *)stream, &e), e);
    }
    // the lists in this library's form, in the scratch: the counts clamped to the capacity [experts], offsets [experts + 1],
    // then perm. The products are given the clamped counts: a count above the capacity names entries the lists do not hold.
    struct Lists { int32_t * counts, * offsets, * perm; int64_t bound; };
    Lists lists(const MatT & m, int rows, const int * counts, const int * groups, int capacity, int experts, StreamT stream) const {
        if (rows <= 0 || m.rows != int64_t(experts) * rows) throw std::invalid_argument("tqmoe adapter: the lists' expert count differs from the bank's");
        Lists l{};
        l.bound = max_assignments > 0 ? max_assignments : int64_t(experts) * capacity;
        const size_t at0 = (size_t(experts) * 4 + 255) / 256 * 256, at1 = at0 + (size_t(experts + 1) * 4 + 255) / 256 * 256;
        if (!scratch || scratch_bytes < at1 + size_t(l.bound) * 4) throw std::invalid_argument("tqmoe adapter: scratch too small for the dispatch lists");
        char * p = static_cast<char *>(scratch);
        l.counts = reinterpret_cast<int32_t *>(p);
        l.offsets = reinterpret_cast<int32_t *>(p + at0);
        l.perm = reinterpret_cast<int32_t *>(p + at1);
        tqmoe_error e = fresh();
        check(tqmoe_lists_from_groups_clamped(counts, groups, capacity, experts, l.counts, l.offsets, l.perm, (void *)stream, &e), e);
        return l;
    }
    bool expert_gemm(const MatT & m, const HalfT * x, Bf16T * y, int rows, const int * counts, const int * groups, int capacity, int experts, int topk,
                     bool per_expert_input, StreamT stream) const override {
        const Lists l = lists(m, rows, counts, groups, capacity, experts, stream);
        tqmoe_error e = fresh();
        const tqmoe_bank b = bank_of(m, rows);
        const int32_t n = int32_t((l.bound + topk - 1) / topk);
        const int32_t rc = tqmoe_expert_gemm(&b, x, TQMOE_F16, l.counts, l.offsets, l.perm, n, topk, topk, 0, per_expert_input ? 1 : 0, y, TQMOE_BF16, (void *)stream, &e);
        if (rc == TQMOE_E_UNSUPPORTED) return false;
        check(rc, e);
        return true;
    }
    bool expert_gemm_gateup(const MatT & g, const MatT & u, const HalfT * x, HalfT * y, int rows, const int * counts, const int * groups, int capacity,
                            int experts, int topk, StreamT stream) const override {
        const Lists l = lists(g, rows, counts, groups, capacity, experts, stream);
        tqmoe_error e = fresh();
        const tqmoe_bank bg = bank_of(g, rows), bu = bank_of(u, rows);
        const int32_t n = int32_t((l.bound + topk - 1) / topk);
        const int32_t rc = tqmoe_expert_gemm_gateup(&bg, &bu, x, TQMOE_F16, l.counts, l.offsets, l.perm, n, topk, topk, 0, y, (void *)stream, &e);
        if (rc == TQMOE_E_UNSUPPORTED) return false;
        check(rc, e);
        return true;
    }
    // expert_gemm_i8 (weight_format.hpp:54-56) on the reference's own operands: xq int8 [rows_in][cols] in natural order, xs fp32
    // [rows_in][cols / 32] (mode 1 a scale per 32 values, mode 2 the token's scale in every entry), xsum the int16 sums per 16
    // values (not read: the minimum term of the formats that have one comes from an operand plane of its own), bf16 rows out.
    // The scratch holds the lists, the rows arranged into operand tiles and their scales (expert_scratch_bytes with int8_mode).
    // false: the format has no int8 grouped product (the caller falls back to expert_gemm), or a mode other than 1 and 2.
    bool expert_gemm_i8(const MatT & m, const int8_t * xq, const float * xs, const int16_t * xsum, Bf16T * y, int rows, const int * counts, const int * groups,
                        int capacity, int experts, int topk, bool per_expert_input, StreamT stream, int mode) const override {
        if (rows <= 0 || m.rows != int64_t(experts) * rows) throw std::invalid_argument("tqmoe adapter: the lists' expert count differs from the bank's");
        if (mode != 1 && mode != 2) return false;
        tqmoe_error e = fresh();
        const tqmoe_bank b = bank_of(m, rows);
        const int64_t bound = max_assignments > 0 ? max_assignments : int64_t(experts) * capacity;
        const int32_t rc = tqmoe_expert_gemm_i8_ref(&b, xq, xs, xsum, y, TQMOE_BF16, counts, groups, capacity, experts, topk, per_expert_input ? 1 : 0, mode, bound,
                                                    scratch, scratch_bytes, (void *)stream, &e);
        if (rc == TQMOE_E_UNSUPPORTED) return false;
        check(rc, e);
        return true;
    }
};

}  // namespace tqmoe_hip

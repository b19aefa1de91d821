// C entry points onto the REFERENCE's own host objects, for validating the restatement in tqmoe_oracle.cpp.
// Built only where the reference tree is present (see Makefile: target ref); the output goes to oracle/_ref/ and is
// test infrastructure like the rest of this directory. This file holds no reference code: it includes the
// reference's headers where they lie and forwards.
#include <cstdint>
#include <cstring>
#include <vector>

#include "experts/moe.hpp"                 // tqllm::moe_route, moe_expert_ffn, moe_combine
#include "experts/cpu_expert_matvec.hpp"   // tqllm::cpu::iq4nl_expert_matvec_*
#include "formats/weight/dequant.hpp"      // tqllm::dequantize_host, half_to_float, float_to_half, e4m3_to_float

extern "C" {

float ref_half_to_float(uint16_t h) { return tqllm::half_to_float(h); }
uint16_t ref_float_to_half(float f) { return tqllm::float_to_half(f); }
float ref_e4m3_to_float(uint8_t b) { return tqllm::e4m3_to_float(b); }

int ref_dequantize(uint32_t type, const void * src, float * dst, int64_t n) {
    try { tqllm::dequantize_host(type, src, dst, n); } catch (...) { return -1; }
    return 0;
}

int ref_route(int gating, int n_expert, int k, int norm_weights, float weight_scale, const float * logits,
              const float * bias, int32_t * ids, float * weights) {
    tqllm::MoeConfig cfg;
    cfg.n_expert = n_expert;
    cfg.n_expert_used = k;
    cfg.gating = static_cast<tqllm::MoeGating>(gating);
    cfg.norm_weights = norm_weights != 0;
    cfg.weight_scale = weight_scale;
    try {
        const tqllm::MoeSelection s = tqllm::moe_route(cfg, logits, bias);
        for (int i = 0; i < k; ++i) { ids[i] = s.ids[size_t(i)]; weights[i] = s.weights[size_t(i)]; }
    } catch (...) { return -1; }
    return 0;
}

void ref_expert_ffn(const float * x, int hidden, const float * w_gate, const float * w_up, const float * w_down, int ff,
                    float swiglu_clamp, int clamp_gate, float * out) {
    tqllm::moe_expert_ffn(x, hidden, w_gate, w_up, w_down, ff, swiglu_clamp, clamp_gate != 0, out);
}

void ref_combine(int k, const float * weights, const float * expert_outs, int hidden, float * out) {
    tqllm::MoeSelection s;
    s.ids.assign(size_t(k), 0);
    s.weights.assign(weights, weights + k);
    tqllm::moe_combine(s, expert_outs, hidden, out);
}

// mode 0 fp32, 1 fp64 accumulate, 2 int8 activations
void ref_iq4nl_matvec(int mode, const uint8_t * W, int rows, int cols, const float * x, int ntok, float * y) {
    const int row_bytes = cols / 32 * 18;
    if (mode == 0) tqllm::cpu::iq4nl_expert_matvec_fp32(W, rows, cols, row_bytes, x, ntok, y);
    else if (mode == 1) tqllm::cpu::iq4nl_expert_matvec_fp64(W, rows, cols, row_bytes, x, ntok, y);
    else tqllm::cpu::iq4nl_expert_matvec_i16(W, rows, cols, row_bytes, x, ntok, y);
}

}  // extern "C"

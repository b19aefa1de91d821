// Prefill-sized expert products of any bank format: the entry of the grouped fp16 GEMM (kernels in
// prefill_f16_kernels.cuh, instantiated per bank format in decode_<format>.hip; IQ4_XS, whose decode-sized kernels are
// its own, here).
#include "prefill_f16_kernels.cuh"

namespace tqmoe {

template struct F16Launch<TQMOE_IQ4_XS>;

namespace {

constexpr int kWideFrom = 64;   // assignments per expert, on average, from which a block takes 128 input rows

void dispatch_f16(uint32_t type, const F16Args & k, bool two, bool wide, dim3 grid, hipStream_t s) {
    switch (type) {
#define X(T) case T: F16Launch<T>::run(k, two, wide, grid, s); break;
        X(TQMOE_IQ4_XS) X(TQMOE_Q4_K) X(TQMOE_IQ3_S) X(TQMOE_IQ4_NL) X(TQMOE_Q8_0) X(TQMOE_Q5_K) X(TQMOE_Q6_K) X(TQMOE_IQ3_XXS) X(TQMOE_IQ2_S)
        X(TQMOE_Q2_K) X(TQMOE_IQ1_S) X(TQMOE_Q4_0) X(TQMOE_Q3_K) X(TQMOE_IQ2_XXS) X(TQMOE_IQ2_XS)
#undef X
        default: F16Launch<TQMOE_NVFP4G>::run(k, two, wide, grid, s); break;
    }
}

}  // namespace

// assignments = total entries of perm; the grid covers the most row blocks the lists can need
int32_t enqueue_gemm_f16(const tqmoe_bank & b0, const tqmoe_bank * b1, const void * x, uint32_t xtype, const int * counts, const int * offsets, const int * perm,
                         int experts, int64_t assignments, int xdiv, void * out, uint32_t out_type, int gateup, int shared_expert, int shared_lim, hipStream_t s, Glu glu) {
    const F16Args k{view(b0), b1 ? view(*b1) : view(b0), x, xtype, counts, offsets, perm, experts, xdiv, out, out_type, gateup, shared_expert, shared_lim, glu};
    const bool wide = assignments >= int64_t(experts) * kWideFrom;   // half a wide tile filled on average
    const int tile = wide ? 128 : 64;                                // input rows of a block
    const int64_t units = assignments / tile + experts;              // sum of ceil(count / tile) never exceeds this
    if (units > 65535) return -1;
    dispatch_f16(b0.type, k, b1 != nullptr, wide, dim3(unsigned((b0.rows + 127) / 128), unsigned(units)), s);
    return 0;
}

}  // namespace tqmoe

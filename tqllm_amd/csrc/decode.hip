// Entry points of the decode-sized expert products and the small element-wise steps around them.
#include "act_image.cuh"
#include "decode_api.cuh"

namespace tqmoe {
int32_t check_bank(const tqmoe_bank * b, const char * what, tqmoe_error * err);  // bank.hip
// prefill_planes.hip (f8: E4M3 operand bytes in place of int8)
int32_t enqueue_quant_rows_i8(const void * x, uint32_t xtype, int64_t rows, int cols, int8_t * q, float * scale, hipStream_t s, bool f8);
int32_t enqueue_gemm_f16(const tqmoe_bank & b0, const tqmoe_bank * b1, const void * x, uint32_t xtype, const int * counts, const int * offsets, const int * perm,
                         int experts, int64_t assignments, int xdiv, void * out, uint32_t out_type, int gateup, int shared_expert, int shared_lim, hipStream_t s, Glu glu);
int64_t grouped_row_tiles(int64_t assignments, int experts);
int64_t grouped_scale_words(int64_t assignments, int experts);
int32_t enqueue_quant_rows_i8_blocks(const void * x, uint32_t xtype, int64_t rows, int cols, int8_t * q, float * scale, int16_t * qsum, hipStream_t s);
int32_t enqueue_gather_rows_i8(const int8_t * rq, const float * rs, int cols, const int * counts, const int * offsets, const int * perm, int experts,
                               int64_t assignments, int xdiv, int8_t * q, float * scale, hipStream_t s, float * block_scale);
int32_t enqueue_group_rows_i8(const void * x, uint32_t xtype, int cols, const int * counts, const int * offsets, const int * perm, int experts,
                              int64_t assignments, int xdiv, int8_t * q, float * scale, hipStream_t s, bool f8, float * block_scale, const float * plan_from);
int32_t enqueue_gather_rows_natural(const int8_t * rq, const float * rs, int cols, const int * counts, const int * offsets, const int * perm, int experts,
                                    int64_t assignments, int xdiv, int8_t * q, float * scale, hipStream_t s, float * block_scale);
bool plane_gemm_has(uint32_t type);
bool plane_gemm_is_fp8(uint32_t type);
int32_t enqueue_plane_gemm(const tqmoe_bank & b0, const tqmoe_bank * b1, const int8_t * xq, const float * xs, const int * counts, const int * offsets,
                           const int * perm, int experts, int64_t assignments, void * out_f16, int gateup, int shared_expert, int shared_lim, hipStream_t s,
                           const float * xbs, Glu glu, int out_bf16, const float * plan_from);
int32_t group_rows_common(const void * x, uint32_t xtype, int32_t cols, const int32_t * counts, const int32_t * offsets, const int32_t * perm, int32_t experts,
                          int64_t assignments, int32_t xdiv, void * q, float * scale, void * stream, tqmoe_error * err, bool f8, const char * what,
                          float * block_scale = nullptr, bool blocks = false, const float * plan_from = nullptr);

int32_t expert_gateup_glu(const tqmoe_bank * gate, const tqmoe_bank * up, const void * x_image, void * act_image, const int32_t * ids, int32_t n,
                          int32_t slots, int32_t topk, int32_t shared_ff, Glu glu, void * stream, tqmoe_error * err);
int32_t gemm_8bit_common(const tqmoe_bank * b0, const tqmoe_bank * b1, const int8_t * xq, const float * xs, const int32_t * counts, const int32_t * offsets,
                         const int32_t * perm, int32_t n, int32_t slots, int32_t topk, int32_t shared_lim, void * out, int gateup, void * stream,
                         tqmoe_error * err, const char * what, bool fp8, const float * block_scale = nullptr, bool blocks = false, Glu glu = Glu{0.f, 0},
                         int out_bf16 = 0, const float * plan_from = nullptr);
int32_t gemm_f16_common(const tqmoe_bank * b0, const tqmoe_bank * b1, const void * x, uint32_t xtype, const int32_t * counts, const int32_t * offsets,
                        const int32_t * perm, int32_t n, int32_t slots, int32_t topk, int32_t shared_lim, int32_t xdiv, void * out, uint32_t otype, int gateup,
                        void * stream, tqmoe_error * err, const char * what, Glu glu = Glu{0.f, 0});

namespace {

__global__ __launch_bounds__(256) void swiglu_k(const float * __restrict__ g, const float * __restrict__ u, float * __restrict__ act, int64_t count, Glu glu) {
    const int64_t i = int64_t(blockIdx.x) * 256 + threadIdx.x;
    if (i < count) {
        float a = g[i], b = u[i];
        glu_clamp_inputs(glu, a, b);
        act[i] = glu_clamp_silu(glu, a / (1.f + expf(-a))) * b;
    }
}

// out[t][j] = sum_s weights[t][s] * routed[t][s][j] (s < topk ascending, rows `slots` per token) + shared_w[t] * shared[t][j]
__device__ __forceinline__ float4 load4(const float * p) { return *reinterpret_cast<const float4 *>(p); }
__device__ __forceinline__ float4 load4(const uint16_t * p) {   // four fp16 values
    const uint2 v = *reinterpret_cast<const uint2 *>(p);
    return make_float4(half_bits_to_float(uint16_t(v.x & 0xFFFFu)), half_bits_to_float(uint16_t(v.x >> 16)), half_bits_to_float(uint16_t(v.y & 0xFFFFu)),
                       half_bits_to_float(uint16_t(v.y >> 16)));
}
// With a residual (bf16 rows, bf16 out) the result is bf16(bf16(sum) + residual): the reference stores the sum as bf16
// (moe_sum) and adds the residual stream to it afterwards (add_sumsq, qwen35_forward.cpp:1248-1250), two roundings.
template <int OT, class RT, int kBatch>
__global__ __launch_bounds__(256) void combine_k(const RT * __restrict__ routed, int slots, const RT * __restrict__ shared, int64_t shared_ld,
                                                 const float * __restrict__ weights, const float * __restrict__ shared_w, void * __restrict__ out, int h, int k,
                                                 int64_t count, const uint16_t * __restrict__ residual) {
    const int64_t i = (int64_t(blockIdx.x) * 256 + threadIdx.x) * 4;   // h is a multiple of 4
    if (i >= count) return;
    const int64_t t = i / h;
    const int j = int(i % h);
    float4 sum = make_float4(0.f, 0.f, 0.f, 0.f);
    // the rows and weights of up to kBatch slots are loaded before the first of them is added: one trip to memory per batch
    // instead of one per slot (the sum keeps the slot order). A few tokens are one chain of trips per thread and take a batch
    // of twelve; many tokens are bound by memory throughput, which the threads' number covers: a batch of one.
    float sw = 0.f;
    float4 sv = make_float4(0.f, 0.f, 0.f, 0.f);
    if (shared) { sw = shared_w[t]; sv = load4(shared + t * shared_ld + j); }
    for (int s0 = 0; s0 < k; s0 += kBatch) {
        float w[kBatch];
        float4 v[kBatch];
#pragma unroll
        for (int q = 0; q < kBatch; ++q)
            if (s0 + q < k) { w[q] = weights[t * k + s0 + q]; v[q] = load4(routed + (t * slots + s0 + q) * h + j); }
#pragma unroll
        for (int q = 0; q < kBatch; ++q)
            if (s0 + q < k) { sum.x += w[q] * v[q].x; sum.y += w[q] * v[q].y; sum.z += w[q] * v[q].z; sum.w += w[q] * v[q].w; }
    }
    if (shared) { sum.x += sw * sv.x; sum.y += sw * sv.y; sum.z += sw * sv.z; sum.w += sw * sv.w; }
    if constexpr (OT == TQMOE_BF16) {
        if (residual) {
            const uint2 r = *reinterpret_cast<const uint2 *>(residual + i);
            sum.x = bf16_bits_to_float(float_to_bf16_bits(sum.x)) + __uint_as_float(r.x << 16);
            sum.y = bf16_bits_to_float(float_to_bf16_bits(sum.y)) + __uint_as_float(r.x & 0xFFFF0000u);
            sum.z = bf16_bits_to_float(float_to_bf16_bits(sum.z)) + __uint_as_float(r.y << 16);
            sum.w = bf16_bits_to_float(float_to_bf16_bits(sum.w)) + __uint_as_float(r.y & 0xFFFF0000u);
        }
    }
    store_out<OT>(out, i, sum.x); store_out<OT>(out, i + 1, sum.y); store_out<OT>(out, i + 2, sum.z); store_out<OT>(out, i + 3, sum.w);
}

__global__ __launch_bounds__(256) void extend_ids_k(const int * __restrict__ ids, int * __restrict__ ext, int topk, int count, int extra) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= count) return;
    const int t = i / (topk + 1), s = i % (topk + 1);
    ext[i] = s < topk ? ids[t * topk + s] : extra;
}

// The reference's dispatch lists (counts [E], groups [E][capacity]) as the lists this library's grouped products read:
// offsets = exclusive scan of the counts, perm = the experts' lists one behind the other. One block; the order inside an
// expert is kept as it is (the reference's device lists are in no particular order, its host lists ascending).
// counts_out (may be null): the counts the lists really hold, min(counts, capacity): what the products must be given, or
// an expert whose count exceeds the capacity would run past its span of perm.
__global__ __launch_bounds__(1024) void lists_from_groups_k(const int * __restrict__ counts, const int * __restrict__ groups, int capacity, int E,
                                                            int * __restrict__ offsets, int * __restrict__ perm, int * __restrict__ counts_out) {
    __shared__ int part[1024];
    extern __shared__ int start[];   // E + 1
    const int tid = threadIdx.x, per = (E + 1023) / 1024, lo = min(tid * per, E), hi = min(lo + per, E);
    int sum = 0;
    for (int e = lo; e < hi; ++e) sum += min(max(counts[e], 0), capacity);
    part[tid] = sum;
    __syncthreads();
    for (int d = 1; d < 1024; d <<= 1) {
        const int v = tid >= d ? part[tid - d] : 0;
        __syncthreads();
        part[tid] += v;
        __syncthreads();
    }
    int base = tid ? part[tid - 1] : 0;
    for (int e = lo; e < hi; ++e) { start[e] = base; base += min(max(counts[e], 0), capacity); }
    if (tid == 1023) start[E] = part[1023];
    __syncthreads();
    for (int e = tid; e <= E; e += 1024) offsets[e] = start[e];
    if (counts_out) for (int e = tid; e < E; e += 1024) counts_out[e] = start[e + 1] - start[e];
    const int lane = tid & 63, wave = tid >> 6;
    for (int e = wave; e < E; e += 16) {   // a wave per expert: coalesced reads of its list
        const int c = start[e + 1] - start[e];
        for (int i = lane; i < c; i += 64) perm[start[e] + i] = groups[int64_t(e) * capacity + i];
    }
}

// The decode grouping maps (kDedupStride ints per group: slot, columns, input row x 8, output row x 8; src/formats/weight/
// quant_kernels.cuh:26-27) as one virtual assignment per map column: its expert (-1 for a column the map does not use, or a
// group whose slot is negative), its input row and its output row.
constexpr int kDedupCols = 8, kDedupStride = 2 + 2 * kDedupCols;
__global__ __launch_bounds__(256) void dedup_expand_k(const int * __restrict__ dmap, int groups, int * __restrict__ ids, int * __restrict__ in_row, int * __restrict__ out_row) {
    const int j = blockIdx.x * 256 + threadIdx.x;
    if (j >= groups * kDedupCols) return;
    const int * e = dmap + int64_t(j / kDedupCols) * kDedupStride;
    const int c = j % kDedupCols;
    const bool live = e[0] >= 0 && c < e[1];
    ids[j] = live ? e[0] : -1;
    in_row[j] = live ? e[2 + c] : -1;
    out_row[j] = live ? e[2 + kDedupCols + c] : -1;
}
// y[out_row[j]] = tmp[j] for the live columns; rows of 2-byte elements (bf16) or 4-byte ones (fp32), `words` dwords a row
__global__ __launch_bounds__(256) void dedup_scatter_k(const uint32_t * __restrict__ tmp0, const uint32_t * __restrict__ tmp1, uint32_t * __restrict__ y0,
                                                       uint32_t * __restrict__ y1, const int * __restrict__ out_row, int words) {
    const int o = out_row[blockIdx.x];
    if (o < 0) return;
    for (int i = threadIdx.x; i < words; i += 256) {
        y0[int64_t(o) * words + i] = tmp0[int64_t(blockIdx.x) * words + i];
        if (tmp1) y1[int64_t(o) * words + i] = tmp1[int64_t(blockIdx.x) * words + i];
    }
}

void dispatch_matvec(uint32_t type, Split sp, int nb, const MatvecArgs & k, hipStream_t s) {
    switch (type) {
        case TQMOE_IQ4_XS: DecodeLaunch<TQMOE_IQ4_XS>::matvec(sp, nb, k, s); break;
        case TQMOE_Q4_K: DecodeLaunch<TQMOE_Q4_K>::matvec(sp, nb, k, s); break;
        case TQMOE_IQ3_S: DecodeLaunch<TQMOE_IQ3_S>::matvec(sp, nb, k, s); break;
        case TQMOE_IQ4_NL: DecodeLaunch<TQMOE_IQ4_NL>::matvec(sp, nb, k, s); break;
        case TQMOE_Q8_0: DecodeLaunch<TQMOE_Q8_0>::matvec(sp, nb, k, s); break;
        case TQMOE_Q5_K: DecodeLaunch<TQMOE_Q5_K>::matvec(sp, nb, k, s); break;
        case TQMOE_Q6_K: DecodeLaunch<TQMOE_Q6_K>::matvec(sp, nb, k, s); break;
        case TQMOE_IQ3_XXS: DecodeLaunch<TQMOE_IQ3_XXS>::matvec(sp, nb, k, s); break;
        case TQMOE_IQ2_S: DecodeLaunch<TQMOE_IQ2_S>::matvec(sp, nb, k, s); break;
        case TQMOE_Q2_K: DecodeLaunch<TQMOE_Q2_K>::matvec(sp, nb, k, s); break;
        case TQMOE_IQ1_S: DecodeLaunch<TQMOE_IQ1_S>::matvec(sp, nb, k, s); break;
        case TQMOE_Q4_0: DecodeLaunch<TQMOE_Q4_0>::matvec(sp, nb, k, s); break;
        case TQMOE_Q3_K: DecodeLaunch<TQMOE_Q3_K>::matvec(sp, nb, k, s); break;
        case TQMOE_IQ2_XXS: DecodeLaunch<TQMOE_IQ2_XXS>::matvec(sp, nb, k, s); break;
        case TQMOE_IQ2_XS: DecodeLaunch<TQMOE_IQ2_XS>::matvec(sp, nb, k, s); break;
        default: DecodeLaunch<TQMOE_NVFP4G>::matvec(sp, nb, k, s); break;
    }
}
void dispatch_gateup(uint32_t type, Split sp, const GateupArgs & k, hipStream_t s) {
    switch (type) {
        case TQMOE_IQ4_XS: DecodeLaunch<TQMOE_IQ4_XS>::gateup(sp, k, s); break;
        case TQMOE_Q4_K: DecodeLaunch<TQMOE_Q4_K>::gateup(sp, k, s); break;
        case TQMOE_IQ3_S: DecodeLaunch<TQMOE_IQ3_S>::gateup(sp, k, s); break;
        case TQMOE_IQ4_NL: DecodeLaunch<TQMOE_IQ4_NL>::gateup(sp, k, s); break;
        case TQMOE_Q8_0: DecodeLaunch<TQMOE_Q8_0>::gateup(sp, k, s); break;
        case TQMOE_Q5_K: DecodeLaunch<TQMOE_Q5_K>::gateup(sp, k, s); break;
        case TQMOE_Q6_K: DecodeLaunch<TQMOE_Q6_K>::gateup(sp, k, s); break;
        case TQMOE_IQ3_XXS: DecodeLaunch<TQMOE_IQ3_XXS>::gateup(sp, k, s); break;
        case TQMOE_IQ2_S: DecodeLaunch<TQMOE_IQ2_S>::gateup(sp, k, s); break;
        case TQMOE_Q2_K: DecodeLaunch<TQMOE_Q2_K>::gateup(sp, k, s); break;
        case TQMOE_IQ1_S: DecodeLaunch<TQMOE_IQ1_S>::gateup(sp, k, s); break;
        case TQMOE_Q4_0: DecodeLaunch<TQMOE_Q4_0>::gateup(sp, k, s); break;
        case TQMOE_Q3_K: DecodeLaunch<TQMOE_Q3_K>::gateup(sp, k, s); break;
        case TQMOE_IQ2_XXS: DecodeLaunch<TQMOE_IQ2_XXS>::gateup(sp, k, s); break;
        case TQMOE_IQ2_XS: DecodeLaunch<TQMOE_IQ2_XS>::gateup(sp, k, s); break;
        default: DecodeLaunch<TQMOE_NVFP4G>::gateup(sp, k, s); break;
    }
}

// one block per expert serves every assignment of that expert when the id list is short enough to scan in the block
constexpr int kScanIds = 2048;
// (a single token's assignments go to different experts: nothing to share, and the scan would only stand in front of the loads)
int dedup_mode(int64_t assignments, int slots) { return assignments > slots && assignments <= kScanIds ? 1 : 0; }

int32_t matvec_common(const tqmoe_bank * b0, const tqmoe_bank * b1, const void * image, void * y0, void * y1, uint32_t ytype, const int32_t * ids,
                      int64_t A, int xdiv, int slots, int topk, int shared_cols, void * stream, tqmoe_error * err, const char * what) {
    if (int32_t rc = check_bank(b0, what, err)) return rc;
    if (b1) {
        if (int32_t rc = check_bank(b1, what, err)) return rc;
        if (b1->type != b0->type || b1->rows != b0->rows || b1->cols != b0->cols || b1->experts != b0->experts)
            return fail(err, TQMOE_E_ARG, "%s: the two banks differ in format or shape", what);
    }
    if (!image || !y0 || (b1 && !y1) || !ids || A <= 0) return fail(err, TQMOE_E_ARG, "%s: invalid shape or pointer", what);
    if (A > 65535) return fail(err, TQMOE_E_ARG, "%s: more than 65535 assignments in one call", what);  // src/formats/weight/quant.cu:73
    if (ytype != TQMOE_F32 && ytype != TQMOE_BF16) return fail(err, TQMOE_E_UNSUPPORTED, "%s: output type must be F32 or BF16", what);
    const Split sp = split_for(b0->cols / 32, A);
    if (sp.m == 0) return fail(err, TQMOE_E_UNSUPPORTED, "%s: cols %d is too wide for the decode kernels", what, b0->cols);
    if (int32_t rc = need_device(err, what)) return rc;
    MatvecArgs k{view(*b0), b1 ? view(*b1) : view(*b0), static_cast<const uint8_t *>(image), y0, y1, ytype, ids, int(A), xdiv, dedup_mode(A, slots), slots, topk, shared_cols};
    dispatch_matvec(b0->type, sp, b1 ? 2 : 1, k, static_cast<hipStream_t>(stream));
    return launched(err, what);
}

}  // namespace
}  // namespace tqmoe

using namespace tqmoe;

extern "C" size_t tqmoe_act_image_bytes(int32_t n, int32_t cols) {
    if (n <= 0 || cols <= 0 || cols % 32) return 0;
    return size_t(n) * size_t(cols / 32) * kImageSubBytes;
}

extern "C" int32_t tqmoe_quant_act(const void * x, uint32_t xtype, int32_t n, int32_t cols, void * image, void * stream, tqmoe_error * err) {
    if (!x || !image || n <= 0 || cols <= 0 || cols % 32) return fail(err, TQMOE_E_ARG, "tqmoe_quant_act: invalid shape or pointer (cols must be a multiple of 32)");
    if (!is_act_type(xtype)) return fail(err, TQMOE_E_UNSUPPORTED, "tqmoe_quant_act: unsupported element type");
    if (int32_t rc = need_device(err, "tqmoe_quant_act")) return rc;
    const unsigned blocks = unsigned((n + 3) / 4);
    const hipStream_t s = static_cast<hipStream_t>(stream);
    uint8_t * img = static_cast<uint8_t *>(image);
    switch (xtype) {
        case TQMOE_F32: quant_act_k<TQMOE_F32><<<blocks, 256, 0, s>>>(x, n, cols, img); break;
        case TQMOE_F16: quant_act_k<TQMOE_F16><<<blocks, 256, 0, s>>>(x, n, cols, img); break;
        default: quant_act_k<TQMOE_BF16><<<blocks, 256, 0, s>>>(x, n, cols, img); break;
    }
    return launched(err, "tqmoe_quant_act");
}

extern "C" int32_t tqmoe_expert_matvec(const tqmoe_bank * bank, const void * image, void * y, uint32_t ytype, const int32_t * ids, int32_t n,
                                       int32_t topk, int32_t per_expert_input, void * stream, tqmoe_error * err) {
    if (n <= 0 || topk <= 0) return fail(err, TQMOE_E_ARG, "tqmoe_expert_matvec: invalid shape");
    return matvec_common(bank, nullptr, image, y, nullptr, ytype, ids, int64_t(n) * topk, per_expert_input ? 1 : topk, 1, 1, 0, stream, err, "tqmoe_expert_matvec");
}

extern "C" int32_t tqmoe_expert_matvec2(const tqmoe_bank * gate, const tqmoe_bank * up, const void * image, void * y_gate, void * y_up, uint32_t ytype,
                                        const int32_t * ids, int32_t n, int32_t topk, void * stream, tqmoe_error * err) {
    if (!up || n <= 0 || topk <= 0) return fail(err, TQMOE_E_ARG, "tqmoe_expert_matvec2: invalid shape or second bank missing");
    return matvec_common(gate, up, image, y_gate, y_up, ytype, ids, int64_t(n) * topk, topk, 1, 1, 0, stream, err, "tqmoe_expert_matvec2");
}

// the decode products on the caller's own rows: the image is made in the caller's scratch and read by the product behind it
static int32_t matvec_rows_common(const tqmoe_bank * b0, const tqmoe_bank * b1, const void * x, uint32_t xtype, void * y0, void * y1, uint32_t ytype,
                                  const int32_t * ids, int32_t n, int32_t topk, int32_t per_expert_input, void * scratch, size_t scratch_bytes, void * stream,
                                  tqmoe_error * err, const char * what) {
    if (!b0 || n <= 0 || topk <= 0 || int64_t(n) * topk > 65535) return fail(err, TQMOE_E_ARG, "%s: invalid shape", what);
    const int32_t rows_in = per_expert_input ? n * topk : n;
    const size_t need = tqmoe_act_image_bytes(rows_in, b0->cols);
    if (!need) return fail(err, TQMOE_E_ARG, "%s: cols must be a positive multiple of 32", what);
    if (!scratch || scratch_bytes < need) return fail(err, TQMOE_E_WORKSPACE, "%s: scratch of %zu bytes needed (tqmoe_act_image_bytes of the input rows)", what, need);
    if (int32_t rc = tqmoe_quant_act(x, xtype, rows_in, b0->cols, scratch, stream, err)) return rc;
    return matvec_common(b0, b1, scratch, y0, y1, ytype, ids, int64_t(n) * topk, per_expert_input ? 1 : topk, 1, 1, 0, stream, err, what);
}

extern "C" int32_t tqmoe_expert_matvec_rows(const tqmoe_bank * bank, const void * x, uint32_t xtype, void * y, uint32_t ytype, const int32_t * ids, int32_t n,
                                            int32_t topk, int32_t per_expert_input, void * scratch, size_t scratch_bytes, void * stream, tqmoe_error * err) {
    return matvec_rows_common(bank, nullptr, x, xtype, y, nullptr, ytype, ids, n, topk, per_expert_input, scratch, scratch_bytes, stream, err, "tqmoe_expert_matvec_rows");
}

extern "C" int32_t tqmoe_expert_matvec2_rows(const tqmoe_bank * gate, const tqmoe_bank * up, const void * x, uint32_t xtype, void * y_gate, void * y_up,
                                             uint32_t ytype, const int32_t * ids, int32_t n, int32_t topk, void * scratch, size_t scratch_bytes, void * stream,
                                             tqmoe_error * err) {
    if (!up) return fail(err, TQMOE_E_ARG, "tqmoe_expert_matvec2_rows: second bank missing");
    return matvec_rows_common(gate, up, x, xtype, y_gate, y_up, ytype, ids, n, topk, 0, scratch, scratch_bytes, stream, err, "tqmoe_expert_matvec2_rows");
}

// scratch of tqmoe_expert_matvec_dedup: ids | input rows | output rows | activation image of the columns | result rows (x2)
namespace {
struct DedupScratch { size_t ids, in_row, out_row, image, y0, y1, total; };
DedupScratch dedup_scratch(int groups, int rows, int cols, uint32_t ytype, bool two) {
    DedupScratch r{};
    size_t o = 0;
    auto take = [&](size_t bytes) { const size_t at = o; o = align_up(o + bytes, 256); return at; };
    const size_t n = size_t(groups) * kDedupCols;
    r.ids = take(n * 4); r.in_row = take(n * 4); r.out_row = take(n * 4);
    r.image = take(tqmoe_act_image_bytes(int32_t(n), cols));
    r.y0 = take(n * rows * elem_bytes(ytype));
    r.y1 = take(two ? n * rows * elem_bytes(ytype) : 0);
    r.total = o;
    return r;
}
}  // namespace

extern "C" size_t tqmoe_expert_matvec_dedup_scratch_bytes(int32_t groups, int32_t rows, int32_t cols, uint32_t ytype, int32_t two_banks) {
    if (groups <= 0 || rows <= 0 || cols <= 0 || cols % 32 || (ytype != TQMOE_F32 && ytype != TQMOE_BF16)) return 0;
    return dedup_scratch(groups, rows, cols, ytype, two_banks != 0).total;
}

extern "C" int32_t tqmoe_expert_matvec_dedup(const tqmoe_bank * bank, const tqmoe_bank * bank2, const void * x, uint32_t xtype, void * y, void * y2, uint32_t ytype,
                                             const int32_t * dmap, int32_t groups, void * scratch, size_t scratch_bytes, void * stream, tqmoe_error * err) {
    const char * what = "tqmoe_expert_matvec_dedup";
    if (int32_t rc = check_bank(bank, what, err)) return rc;
    if (!x || !y || (bank2 && !y2) || !dmap || groups <= 0 || int64_t(groups) * kDedupCols > 65535) return fail(err, TQMOE_E_ARG, "%s: invalid shape or pointer", what);
    if (!is_act_type(xtype) || (ytype != TQMOE_F32 && ytype != TQMOE_BF16)) return fail(err, TQMOE_E_UNSUPPORTED, "%s: unsupported element type", what);
    const DedupScratch r = dedup_scratch(groups, bank->rows, bank->cols, ytype, bank2 != nullptr);
    if (!scratch || scratch_bytes < r.total) return fail(err, TQMOE_E_WORKSPACE, "%s: scratch of %zu bytes needed", what, r.total);
    if (int32_t rc = need_device(err, what)) return rc;
    uint8_t * ws = static_cast<uint8_t *>(scratch);
    int32_t * ids = reinterpret_cast<int32_t *>(ws + r.ids), * in_row = reinterpret_cast<int32_t *>(ws + r.in_row), * out_row = reinterpret_cast<int32_t *>(ws + r.out_row);
    const int n = groups * kDedupCols;
    const hipStream_t s = static_cast<hipStream_t>(stream);
    dedup_expand_k<<<unsigned((n + 255) / 256), 256, 0, s>>>(dmap, groups, ids, in_row, out_row);
    const unsigned qblocks = unsigned((n + 3) / 4);
    switch (xtype) {
        case TQMOE_F32: quant_act_k<TQMOE_F32><<<qblocks, 256, 0, s>>>(x, n, bank->cols, ws + r.image, in_row); break;
        case TQMOE_F16: quant_act_k<TQMOE_F16><<<qblocks, 256, 0, s>>>(x, n, bank->cols, ws + r.image, in_row); break;
        default: quant_act_k<TQMOE_BF16><<<qblocks, 256, 0, s>>>(x, n, bank->cols, ws + r.image, in_row); break;
    }
    if (int32_t rc = launched(err, what)) return rc;
    // a virtual assignment per map column, one input row each; the kernels serve an expert's columns together as they do for ids
    if (int32_t rc = matvec_common(bank, bank2, ws + r.image, ws + r.y0, bank2 ? ws + r.y1 : nullptr, ytype, ids, n, 1, 1, 1, 0, stream, err, what)) return rc;
    const int words = int(size_t(bank->rows) * elem_bytes(ytype) / 4);
    if (size_t(bank->rows) * elem_bytes(ytype) % 4) return fail(err, TQMOE_E_ARG, "%s: rows must make whole dwords", what);
    dedup_scatter_k<<<unsigned(n), 256, 0, s>>>(reinterpret_cast<const uint32_t *>(ws + r.y0), bank2 ? reinterpret_cast<const uint32_t *>(ws + r.y1) : nullptr,
                                                static_cast<uint32_t *>(y), static_cast<uint32_t *>(y2), out_row, words);
    return launched(err, what);
}

extern "C" int32_t tqmoe_lists_from_groups_clamped(const int32_t * counts, const int32_t * groups, int32_t capacity, int32_t experts, int32_t * counts_out,
                                                   int32_t * offsets, int32_t * perm, void * stream, tqmoe_error * err) {
    if (!counts || !groups || !offsets || !perm || capacity <= 0 || experts <= 0 || experts > 4096)
        return fail(err, TQMOE_E_ARG, "tqmoe_lists_from_groups: invalid shape or pointer");
    if (int32_t rc = need_device(err, "tqmoe_lists_from_groups")) return rc;
    lists_from_groups_k<<<1, 1024, size_t(experts + 1) * sizeof(int), static_cast<hipStream_t>(stream)>>>(counts, groups, capacity, experts, offsets, perm, counts_out);
    return launched(err, "tqmoe_lists_from_groups");
}

extern "C" int32_t tqmoe_lists_from_groups(const int32_t * counts, const int32_t * groups, int32_t capacity, int32_t experts, int32_t * offsets, int32_t * perm,
                                           void * stream, tqmoe_error * err) {
    return tqmoe_lists_from_groups_clamped(counts, groups, capacity, experts, nullptr, offsets, perm, stream, err);
}

extern "C" int32_t tqmoe_extend_ids(const int32_t * ids, int32_t * out, int32_t topk, int32_t n, int32_t extra, void * stream, tqmoe_error * err) {
    if (!ids || !out || topk <= 0 || n <= 0 || int64_t(n) * (topk + 1) > 0x7FFFFFFF) return fail(err, TQMOE_E_ARG, "tqmoe_extend_ids: invalid shape or pointer");
    if (int32_t rc = need_device(err, "tqmoe_extend_ids")) return rc;
    const int count = n * (topk + 1);
    extend_ids_k<<<unsigned((count + 255) / 256), 256, 0, static_cast<hipStream_t>(stream)>>>(ids, out, topk, count, extra);
    return launched(err, "tqmoe_extend_ids");
}

// The gate / up products of the three paths with the optional clamp of the SwiGLU inputs (the layer's swiglu_clamp); the
// C entry points are these without a clamp.
int32_t tqmoe::expert_gateup_glu(const tqmoe_bank * gate, const tqmoe_bank * up, const void * x_image, void * act_image, const int32_t * ids, int32_t n,
                                 int32_t slots, int32_t topk, int32_t shared_ff, Glu glu, void * stream, tqmoe_error * err) {
    const char * what = "tqmoe_expert_gateup";
    if (int32_t rc = check_bank(gate, what, err)) return rc;
    if (int32_t rc = check_bank(up, what, err)) return rc;
    if (up->type != gate->type || up->rows != gate->rows || up->cols != gate->cols || up->experts != gate->experts)
        return fail(err, TQMOE_E_ARG, "%s: the two banks differ in format or shape", what);
    if (!x_image || !act_image || !ids || n <= 0 || topk <= 0 || slots < topk || gate->rows % 32) return fail(err, TQMOE_E_ARG, "%s: invalid shape or pointer", what);
    if (slots > topk && (shared_ff <= 0 || shared_ff > gate->rows || shared_ff % 32)) return fail(err, TQMOE_E_ARG, "%s: invalid shared_ff", what);
    const int64_t A = int64_t(n) * slots;
    if (A > 65535) return fail(err, TQMOE_E_ARG, "%s: more than 65535 assignments in one call", what);
    const Split sp = split_for(gate->cols / 32, A);
    if (sp.m == 0) return fail(err, TQMOE_E_UNSUPPORTED, "%s: cols %d is too wide for the decode kernels", what, gate->cols);
    if (int32_t rc = need_device(err, what)) return rc;
    GateupArgs k{view(*gate), view(*up), static_cast<const uint8_t *>(x_image), static_cast<uint8_t *>(act_image), ids, int(A), slots, topk, shared_ff, dedup_mode(A, slots), glu};
    dispatch_gateup(gate->type, sp, k, static_cast<hipStream_t>(stream));
    return launched(err, what);
}

extern "C" int32_t tqmoe_expert_gateup(const tqmoe_bank * gate, const tqmoe_bank * up, const void * x_image, void * act_image, const int32_t * ids,
                                       int32_t n, int32_t slots, int32_t topk, int32_t shared_ff, void * stream, tqmoe_error * err) {
    return expert_gateup_glu(gate, up, x_image, act_image, ids, n, slots, topk, shared_ff, Glu{0.f, 0}, stream, err);
}

extern "C" int32_t tqmoe_expert_down(const tqmoe_bank * down, const void * act_image, float * y, const int32_t * ids, int32_t n, int32_t slots,
                                     int32_t topk, int32_t shared_ff, void * stream, tqmoe_error * err) {
    const char * what = "tqmoe_expert_down";
    if (n <= 0 || topk <= 0 || slots < topk) return fail(err, TQMOE_E_ARG, "%s: invalid shape", what);
    if (slots > topk && (!down || shared_ff <= 0 || shared_ff > down->cols || shared_ff % 32)) return fail(err, TQMOE_E_ARG, "%s: invalid shared_ff", what);
    if (slots > topk && down->type == TQMOE_IQ4_XS && shared_ff % 256) return fail(err, TQMOE_E_UNSUPPORTED, "%s: IQ4_XS needs shared_ff in whole 256-weight blocks", what);
    return matvec_common(down, nullptr, act_image, y, nullptr, TQMOE_F32, ids, int64_t(n) * slots, 1, slots, topk, shared_ff, stream, err, what);
}

extern "C" int32_t tqmoe_swiglu_clamped(const float * gate, const float * up, float * act, int64_t count, float swiglu_clamp, int32_t clamp_gate, void * stream,
                                        tqmoe_error * err) {
    if (!gate || !up || !act || count <= 0 || (count + 255) / 256 > 0x7FFFFFFF) return fail(err, TQMOE_E_ARG, "tqmoe_swiglu: invalid size or pointer");
    if (int32_t rc = need_device(err, "tqmoe_swiglu")) return rc;
    swiglu_k<<<unsigned((count + 255) / 256), 256, 0, static_cast<hipStream_t>(stream)>>>(gate, up, act, count, Glu{swiglu_clamp, clamp_gate ? 1 : 0});
    return launched(err, "tqmoe_swiglu");
}

extern "C" int32_t tqmoe_swiglu(const float * gate, const float * up, float * act, int64_t count, void * stream, tqmoe_error * err) {
    return tqmoe_swiglu_clamped(gate, up, act, count, 0.f, 0, stream, err);
}

template <class RT>
static int32_t combine_common(const RT * routed, int32_t slots, const RT * shared, int64_t shared_ld, const float * weights, const float * shared_weights,
                              void * out, uint32_t otype, int32_t hidden, int32_t topk, int32_t n, void * stream, tqmoe_error * err,
                              const uint16_t * residual = nullptr) {
    if (!routed || !weights || !out || hidden <= 0 || hidden % 4 || topk <= 0 || slots < topk || n <= 0 || (shared && (!shared_weights || shared_ld % 4)))
        return fail(err, TQMOE_E_ARG, "tqmoe_combine: invalid shape or pointer (hidden must be a multiple of 4)");
    if (otype != TQMOE_F32 && otype != TQMOE_BF16) return fail(err, TQMOE_E_UNSUPPORTED, "tqmoe_combine: output type must be F32 or BF16");
    if (int32_t rc = need_device(err, "tqmoe_combine")) return rc;
    const int64_t count = int64_t(n) * hidden;
    const unsigned blocks = unsigned((count / 4 + 255) / 256);
    const hipStream_t s = static_cast<hipStream_t>(stream);
    if (residual && otype != TQMOE_BF16) return fail(err, TQMOE_E_UNSUPPORTED, "tqmoe_combine: a residual is added to BF16 output only");
    const bool few = n <= 64;
    if (otype == TQMOE_F32) {
        if (few) combine_k<TQMOE_F32, RT, 12><<<blocks, 256, 0, s>>>(routed, slots, shared, shared_ld, weights, shared_weights, out, hidden, topk, count, nullptr);
        else combine_k<TQMOE_F32, RT, 1><<<blocks, 256, 0, s>>>(routed, slots, shared, shared_ld, weights, shared_weights, out, hidden, topk, count, nullptr);
    } else {
        if (few) combine_k<TQMOE_BF16, RT, 12><<<blocks, 256, 0, s>>>(routed, slots, shared, shared_ld, weights, shared_weights, out, hidden, topk, count, residual);
        else combine_k<TQMOE_BF16, RT, 1><<<blocks, 256, 0, s>>>(routed, slots, shared, shared_ld, weights, shared_weights, out, hidden, topk, count, residual);
    }
    return launched(err, "tqmoe_combine");
}

extern "C" int32_t tqmoe_combine_residual(const void * routed, uint32_t rtype, int32_t slots, const void * shared, int64_t shared_ld, const float * weights,
                                          const float * shared_weights, const void * residual, void * out, int32_t hidden, int32_t topk, int32_t n,
                                          void * stream, tqmoe_error * err) {
    if (!residual) return fail(err, TQMOE_E_ARG, "tqmoe_combine_residual: residual rows missing");
    if (rtype == TQMOE_F32)
        return combine_common<float>(static_cast<const float *>(routed), slots, static_cast<const float *>(shared), shared_ld, weights, shared_weights, out,
                                     TQMOE_BF16, hidden, topk, n, stream, err, static_cast<const uint16_t *>(residual));
    if (rtype == TQMOE_F16)
        return combine_common<uint16_t>(static_cast<const uint16_t *>(routed), slots, static_cast<const uint16_t *>(shared), shared_ld, weights, shared_weights,
                                        out, TQMOE_BF16, hidden, topk, n, stream, err, static_cast<const uint16_t *>(residual));
    return fail(err, TQMOE_E_UNSUPPORTED, "tqmoe_combine_residual: routed rows are F32 or F16");
}

extern "C" int32_t tqmoe_combine_strided(const float * routed, int32_t slots, const float * shared, int64_t shared_ld, const float * weights,
                                         const float * shared_weights, void * out, uint32_t otype, int32_t hidden, int32_t topk, int32_t n, void * stream,
                                         tqmoe_error * err) {
    return combine_common<float>(routed, slots, shared, shared_ld, weights, shared_weights, out, otype, hidden, topk, n, stream, err);
}

extern "C" int32_t tqmoe_combine_strided_f16(const void * routed, int32_t slots, const void * shared, int64_t shared_ld, const float * weights,
                                             const float * shared_weights, void * out, uint32_t otype, int32_t hidden, int32_t topk, int32_t n,
                                             void * stream, tqmoe_error * err) {
    return combine_common<uint16_t>(static_cast<const uint16_t *>(routed), slots, static_cast<const uint16_t *>(shared), shared_ld, weights, shared_weights, out,
                                    otype, hidden, topk, n, stream, err);
}

extern "C" int32_t tqmoe_combine(const float * routed, const float * shared, const float * weights, const float * shared_weights, void * out,
                                 uint32_t otype, int32_t hidden, int32_t topk, int32_t n, void * stream, tqmoe_error * err) {
    return tqmoe_combine_strided(routed, topk, shared, hidden, weights, shared_weights, out, otype, hidden, topk, n, stream, err);
}

static int32_t quant_rows_common(const void * x, uint32_t xtype, int64_t rows, int32_t cols, void * q, float * scale, void * stream, tqmoe_error * err, bool f8,
                                 const char * what) {
    if (!x || !q || !scale || rows <= 0 || cols <= 0 || cols % 32 || (rows + 3) / 4 > 0x7FFFFFFF) return fail(err, TQMOE_E_ARG, "%s: invalid shape or pointer", what);
    if (!is_act_type(xtype)) return fail(err, TQMOE_E_UNSUPPORTED, "%s: unsupported element type", what);
    if (int32_t rc = need_device(err, what)) return rc;
    enqueue_quant_rows_i8(x, xtype, rows, cols, static_cast<int8_t *>(q), scale, static_cast<hipStream_t>(stream), f8);
    return launched(err, what);
}

extern "C" int32_t tqmoe_quant_rows_i8(const void * x, uint32_t xtype, int64_t rows, int32_t cols, int8_t * q, float * scale, void * stream, tqmoe_error * err) {
    return quant_rows_common(x, xtype, rows, cols, q, scale, stream, err, false, "tqmoe_quant_rows_i8");
}

extern "C" int32_t tqmoe_quant_rows_fp8(const void * x, uint32_t xtype, int64_t rows, int32_t cols, uint8_t * q, float * scale, void * stream, tqmoe_error * err) {
    return quant_rows_common(x, xtype, rows, cols, q, scale, stream, err, true, "tqmoe_quant_rows_fp8");
}

extern "C" int32_t tqmoe_quant_rows_i8_blocks(const void * x, uint32_t xtype, int64_t rows, int32_t cols, int8_t * q, float * scales, int16_t * qsum, void * stream,
                                              tqmoe_error * err) {
    const char * what = "tqmoe_quant_rows_i8_blocks";
    if (!x || !q || !scales || rows <= 0 || cols <= 0 || cols % 32 || (rows + 3) / 4 > 0x7FFFFFFF) return fail(err, TQMOE_E_ARG, "%s: invalid shape or pointer", what);
    if (!is_act_type(xtype)) return fail(err, TQMOE_E_UNSUPPORTED, "%s: unsupported element type", what);
    if (int32_t rc = need_device(err, what)) return rc;
    enqueue_quant_rows_i8_blocks(x, xtype, rows, cols, q, scales, qsum, static_cast<hipStream_t>(stream));
    return launched(err, what);
}

extern "C" int64_t tqmoe_grouped_block_scale_words(int64_t assignments, int32_t experts, int32_t cols) {
    return assignments > 0 && experts > 0 && cols > 0 && cols % 32 == 0 ? grouped_row_tiles(assignments, experts) * 32 * (cols / 32) : 0;
}

extern "C" int64_t tqmoe_grouped_rows(int64_t assignments, int32_t experts) {
    return assignments > 0 && experts > 0 ? grouped_row_tiles(assignments, experts) * 32 : 0;
}

extern "C" int64_t tqmoe_grouped_scale_words(int64_t assignments, int32_t experts) {
    return assignments > 0 && experts > 0 ? grouped_scale_words(assignments, experts) : 0;
}

int32_t tqmoe::group_rows_common(const void * x, uint32_t xtype, int32_t cols, const int32_t * counts, const int32_t * offsets, const int32_t * perm, int32_t experts,
                                 int64_t assignments, int32_t xdiv, void * q, float * scale, void * stream, tqmoe_error * err, bool f8, const char * what,
                                 float * block_scale, bool blocks, const float * plan_from) {
    if (blocks && !block_scale) return fail(err, TQMOE_E_ARG, "%s: block scales missing", what);
    if (!x || !counts || !offsets || !perm || !q || !scale || cols <= 0 || cols % 32 || experts <= 0 || experts > 4096 || assignments <= 0 || xdiv <= 0 ||
        grouped_row_tiles(assignments, experts) > 0x7FFFFFFF)
        return fail(err, TQMOE_E_ARG, "%s: invalid shape or pointer", what);
    if (!is_act_type(xtype)) return fail(err, TQMOE_E_UNSUPPORTED, "%s: unsupported element type", what);
    if (int32_t rc = need_device(err, what)) return rc;
    enqueue_group_rows_i8(x, xtype, cols, counts, offsets, perm, experts, assignments, xdiv, static_cast<int8_t *>(q), scale, static_cast<hipStream_t>(stream), f8,
                          block_scale, plan_from);
    return launched(err, what);
}

extern "C" int32_t tqmoe_group_rows_i8_blocks(const void * x, uint32_t xtype, int32_t cols, const int32_t * counts, const int32_t * offsets, const int32_t * perm,
                                              int32_t experts, int64_t assignments, int32_t xdiv, int8_t * q, float * scale, float * block_scale, void * stream,
                                              tqmoe_error * err) {
    return group_rows_common(x, xtype, cols, counts, offsets, perm, experts, assignments, xdiv, q, scale, stream, err, false, "tqmoe_group_rows_i8_blocks", block_scale, true);
}

extern "C" int32_t tqmoe_group_rows_i8(const void * x, uint32_t xtype, int32_t cols, const int32_t * counts, const int32_t * offsets, const int32_t * perm,
                                       int32_t experts, int64_t assignments, int32_t xdiv, int8_t * q, float * scale, void * stream, tqmoe_error * err) {
    return group_rows_common(x, xtype, cols, counts, offsets, perm, experts, assignments, xdiv, q, scale, stream, err, false, "tqmoe_group_rows_i8");
}

extern "C" int32_t tqmoe_group_rows_fp8(const void * x, uint32_t xtype, int32_t cols, const int32_t * counts, const int32_t * offsets, const int32_t * perm,
                                        int32_t experts, int64_t assignments, int32_t xdiv, uint8_t * q, float * scale, void * stream, tqmoe_error * err) {
    return group_rows_common(x, xtype, cols, counts, offsets, perm, experts, assignments, xdiv, q, scale, stream, err, true, "tqmoe_group_rows_fp8");
}

static int32_t gather_rows_common(const int8_t * rows_q, const float * rows_scale, int32_t cols, const int32_t * counts, const int32_t * offsets,
                                  const int32_t * perm, int32_t experts, int64_t assignments, int32_t xdiv, int8_t * q, float * scale, float * block_scale,
                                  bool blocks, void * stream, tqmoe_error * err, const char * what) {
    if (!rows_q || !rows_scale || !counts || !offsets || !perm || !q || !scale || (blocks && !block_scale) || cols <= 0 || cols % 32 || experts <= 0 ||
        experts > 4096 || assignments <= 0 || xdiv <= 0 || grouped_row_tiles(assignments, experts) > 0x7FFFFFFF)
        return fail(err, TQMOE_E_ARG, "%s: invalid shape or pointer", what);
    if (int32_t rc = need_device(err, what)) return rc;
    enqueue_gather_rows_i8(rows_q, rows_scale, cols, counts, offsets, perm, experts, assignments, xdiv, q, scale, static_cast<hipStream_t>(stream), block_scale);
    return launched(err, what);
}

extern "C" int32_t tqmoe_gather_rows_i8(const int8_t * rows_q, const float * rows_scale, int32_t cols, const int32_t * counts, const int32_t * offsets,
                                        const int32_t * perm, int32_t experts, int64_t assignments, int32_t xdiv, int8_t * q, float * scale, void * stream,
                                        tqmoe_error * err) {
    return gather_rows_common(rows_q, rows_scale, cols, counts, offsets, perm, experts, assignments, xdiv, q, scale, nullptr, false, stream, err, "tqmoe_gather_rows_i8");
}

extern "C" int32_t tqmoe_gather_rows_i8_blocks(const int8_t * rows_q, const float * rows_scales, int32_t cols, const int32_t * counts, const int32_t * offsets,
                                               const int32_t * perm, int32_t experts, int64_t assignments, int32_t xdiv, int8_t * q, float * scale,
                                               float * block_scale, void * stream, tqmoe_error * err) {
    return gather_rows_common(rows_q, rows_scales, cols, counts, offsets, perm, experts, assignments, xdiv, q, scale, block_scale, true, stream, err,
                              "tqmoe_gather_rows_i8_blocks");
}

int32_t tqmoe::gemm_8bit_common(const tqmoe_bank * b0, const tqmoe_bank * b1, const int8_t * xq, const float * xs, const int32_t * counts, const int32_t * offsets,
                           const int32_t * perm, int32_t n, int32_t slots, int32_t topk, int32_t shared_lim, void * out, int gateup, void * stream,
                           tqmoe_error * err, const char * what, bool fp8, const float * block_scale, bool blocks, Glu glu, int out_bf16, const float * plan_from) {
    if (blocks && !block_scale) return fail(err, TQMOE_E_ARG, "%s: block scales missing", what);
    if (int32_t rc = check_bank(b0, what, err)) return rc;
    if (b1) {
        if (int32_t rc = check_bank(b1, what, err)) return rc;
        if (b1->type != b0->type || b1->rows != b0->rows || b1->cols != b0->cols || b1->experts != b0->experts)
            return fail(err, TQMOE_E_ARG, "%s: the two banks differ in format or shape", what);
    }
    if (!plane_gemm_has(b0->type) || plane_gemm_is_fp8(b0->type) != fp8)
        return fail(err, TQMOE_E_UNSUPPORTED, "%s: no %s grouped product for bank type %u (false in the reference's terms: use the fp16 grouped or the decode products)", what,
                    fp8 ? "fp8" : "int8", b0->type);
    if (b0->cols % 256 || b0->rows % 32) return fail(err, TQMOE_E_UNSUPPORTED, "%s: the bank's rows must be a multiple of 32 and its columns of 256", what);
    if (!xq || !xs || !counts || !offsets || !perm || !out || n <= 0 || topk <= 0 || slots < topk) return fail(err, TQMOE_E_ARG, "%s: invalid shape or pointer", what);
    const int lim_max = gateup ? b0->rows : b0->cols;
    if (slots > topk && (shared_lim <= 0 || shared_lim > lim_max || shared_lim % 256)) return fail(err, TQMOE_E_ARG, "%s: shared_lim must be a multiple of 256 within the bank", what);
    if (b0->experts > 4096) return fail(err, TQMOE_E_ARG, "%s: more than 4096 experts", what);
    if (int32_t rc = need_device(err, what)) return rc;
    const int shared_expert = slots > topk ? b0->experts - 1 : -1;
    if (enqueue_plane_gemm(*b0, b1, xq, xs, counts, offsets, perm, b0->experts, int64_t(n) * slots, out, gateup, shared_expert, shared_lim,
                           static_cast<hipStream_t>(stream), block_scale, glu, out_bf16, plan_from))
        return fail(err, TQMOE_E_ARG, "%s: too many assignments for one call", what);
    return launched(err, what);
}

extern "C" int32_t tqmoe_expert_gemm_gateup_i8(const tqmoe_bank * gate, const tqmoe_bank * up, const int8_t * xq, const float * xs, const int32_t * counts,
                                               const int32_t * offsets, const int32_t * perm, int32_t n, int32_t slots, int32_t topk, int32_t shared_lim,
                                               void * act_f16, void * stream, tqmoe_error * err) {
    if (!up) return fail(err, TQMOE_E_ARG, "tqmoe_expert_gemm_gateup_i8: second bank missing");
    return gemm_8bit_common(gate, up, xq, xs, counts, offsets, perm, n, slots, topk, shared_lim, act_f16, 1, stream, err, "tqmoe_expert_gemm_gateup_i8", false);
}

extern "C" int32_t tqmoe_expert_gemm_i8(const tqmoe_bank * bank, const int8_t * xq, const float * xs, const int32_t * counts, const int32_t * offsets,
                                        const int32_t * perm, int32_t n, int32_t slots, int32_t topk, int32_t shared_lim, void * y_f16, void * stream,
                                        tqmoe_error * err) {
    return gemm_8bit_common(bank, nullptr, xq, xs, counts, offsets, perm, n, slots, topk, shared_lim, y_f16, 0, stream, err, "tqmoe_expert_gemm_i8", false);
}

// scratch of tqmoe_expert_gemm_i8_ref: clamped counts | offsets | perm | grouped rows | their scales and index | block scales
namespace {
struct RefScratch { size_t counts, offsets, perm, q, scale, block_scale, total; };
RefScratch ref_scratch(int experts, int64_t bound, int cols, int mode) {
    RefScratch r{};
    size_t o = 0;
    auto take = [&](size_t bytes) { const size_t at = o; o = align_up(o + bytes, 256); return at; };
    r.counts = take(size_t(experts) * 4);
    r.offsets = take(size_t(experts + 1) * 4);
    r.perm = take(size_t(bound) * 4);
    r.q = take(size_t(tqmoe_grouped_rows(bound, experts)) * size_t(cols));
    r.scale = take(size_t(tqmoe_grouped_scale_words(bound, experts)) * 4);
    r.block_scale = take(mode == 1 ? size_t(tqmoe_grouped_block_scale_words(bound, experts, cols)) * 4 : 0);
    r.total = o;
    return r;
}
}  // namespace

extern "C" size_t tqmoe_expert_gemm_i8_ref_scratch_bytes(int32_t experts, int64_t max_assignments, int32_t cols, int32_t mode) {
    if (experts <= 0 || experts > 4096 || max_assignments <= 0 || cols <= 0 || cols % 32 || (mode != 1 && mode != 2)) return 0;
    return ref_scratch(experts, max_assignments, cols, mode).total;
}

extern "C" int32_t tqmoe_expert_gemm_i8_ref(const tqmoe_bank * bank, const int8_t * xq, const float * xs, const int16_t * xsum, void * y, uint32_t ytype,
                                            const int32_t * counts, const int32_t * groups, int32_t capacity, int32_t experts, int32_t topk,
                                            int32_t per_expert_input, int32_t mode, int64_t max_assignments, void * scratch, size_t scratch_bytes,
                                            void * stream, tqmoe_error * err) {
    const char * what = "tqmoe_expert_gemm_i8_ref";
    (void)xsum;   // the sums of q per 16 values feed the reference's minimum term; the products here take that term from a plane of their own
    if (int32_t rc = check_bank(bank, what, err)) return rc;
    if (mode != 1 && mode != 2) return fail(err, TQMOE_E_UNSUPPORTED, "%s: mode %d (1: a scale per 32 values, 2: per token)", what, mode);
    if (ytype != TQMOE_BF16 && ytype != TQMOE_F16) return fail(err, TQMOE_E_UNSUPPORTED, "%s: output rows are BF16 or F16", what);
    if (!xq || !xs || !y || !counts || !groups || capacity <= 0 || experts <= 0 || topk <= 0 || max_assignments <= 0)
        return fail(err, TQMOE_E_ARG, "%s: invalid shape or pointer", what);
    if (experts != bank->experts) return fail(err, TQMOE_E_ARG, "%s: %d lists for a bank of %d experts", what, experts, bank->experts);
    if (max_assignments > int64_t(experts) * capacity) max_assignments = int64_t(experts) * capacity;
    const RefScratch r = ref_scratch(experts, max_assignments, bank->cols, mode);
    if (!scratch || scratch_bytes < r.total) return fail(err, TQMOE_E_WORKSPACE, "%s: scratch of %zu bytes needed", what, r.total);
    if (!plane_gemm_has(bank->type) || plane_gemm_is_fp8(bank->type))
        return fail(err, TQMOE_E_UNSUPPORTED, "%s: no int8 grouped product for bank type %u (false in the reference's terms)", what, bank->type);
    uint8_t * ws = static_cast<uint8_t *>(scratch);
    int32_t * cc = reinterpret_cast<int32_t *>(ws + r.counts), * offsets = reinterpret_cast<int32_t *>(ws + r.offsets), * perm = reinterpret_cast<int32_t *>(ws + r.perm);
    int8_t * q = reinterpret_cast<int8_t *>(ws + r.q);
    float * scale = reinterpret_cast<float *>(ws + r.scale), * bscale = mode == 1 ? reinterpret_cast<float *>(ws + r.block_scale) : nullptr;
    if (int32_t rc = tqmoe_lists_from_groups_clamped(counts, groups, capacity, experts, cc, offsets, perm, stream, err)) return rc;
    enqueue_gather_rows_natural(xq, xs, bank->cols, cc, offsets, perm, experts, max_assignments, per_expert_input ? 1 : topk, q, scale,
                                static_cast<hipStream_t>(stream), bscale);
    if (int32_t rc = launched(err, what)) return rc;
    // (n x slots only bounds the listed assignments: it fixes where the index behind the scales lies)
    return gemm_8bit_common(bank, nullptr, q, scale, cc, offsets, perm, 1, int32_t(max_assignments), int32_t(max_assignments), 0, y, 0, stream, err, what, false,
                            bscale, mode == 1, Glu{0.f, 0}, ytype == TQMOE_BF16);
}

extern "C" int32_t tqmoe_expert_gemm_gateup_i8_blocks(const tqmoe_bank * gate, const tqmoe_bank * up, const int8_t * xq, const float * xs, const float * block_scale,
                                                      const int32_t * counts, const int32_t * offsets, const int32_t * perm, int32_t n, int32_t slots, int32_t topk,
                                                      int32_t shared_lim, void * act_f16, void * stream, tqmoe_error * err) {
    if (!up) return fail(err, TQMOE_E_ARG, "tqmoe_expert_gemm_gateup_i8_blocks: second bank missing");
    return gemm_8bit_common(gate, up, xq, xs, counts, offsets, perm, n, slots, topk, shared_lim, act_f16, 1, stream, err, "tqmoe_expert_gemm_gateup_i8_blocks", false,
                       block_scale, true);
}

extern "C" int32_t tqmoe_expert_gemm_i8_blocks(const tqmoe_bank * bank, const int8_t * xq, const float * xs, const float * block_scale, const int32_t * counts,
                                               const int32_t * offsets, const int32_t * perm, int32_t n, int32_t slots, int32_t topk, int32_t shared_lim,
                                               void * y_f16, void * stream, tqmoe_error * err) {
    return gemm_8bit_common(bank, nullptr, xq, xs, counts, offsets, perm, n, slots, topk, shared_lim, y_f16, 0, stream, err, "tqmoe_expert_gemm_i8_blocks", false, block_scale,
                       true);
}

extern "C" int32_t tqmoe_expert_gemm_gateup_fp8(const tqmoe_bank * gate, const tqmoe_bank * up, const uint8_t * xq, const float * xs, const int32_t * counts,
                                                const int32_t * offsets, const int32_t * perm, int32_t n, int32_t slots, int32_t topk, int32_t shared_lim,
                                                void * act_f16, void * stream, tqmoe_error * err) {
    if (!up) return fail(err, TQMOE_E_ARG, "tqmoe_expert_gemm_gateup_fp8: second bank missing");
    return gemm_8bit_common(gate, up, reinterpret_cast<const int8_t *>(xq), xs, counts, offsets, perm, n, slots, topk, shared_lim, act_f16, 1, stream, err,
                       "tqmoe_expert_gemm_gateup_fp8", true);
}

extern "C" int32_t tqmoe_expert_gemm_fp8(const tqmoe_bank * bank, const uint8_t * xq, const float * xs, const int32_t * counts, const int32_t * offsets,
                                         const int32_t * perm, int32_t n, int32_t slots, int32_t topk, int32_t shared_lim, void * y_f16, void * stream,
                                         tqmoe_error * err) {
    return gemm_8bit_common(bank, nullptr, reinterpret_cast<const int8_t *>(xq), xs, counts, offsets, perm, n, slots, topk, shared_lim, y_f16, 0, stream, err,
                       "tqmoe_expert_gemm_fp8", true);
}

int32_t tqmoe::gemm_f16_common(const tqmoe_bank * b0, const tqmoe_bank * b1, const void * x, uint32_t xtype, const int32_t * counts, const int32_t * offsets,
                               const int32_t * perm, int32_t n, int32_t slots, int32_t topk, int32_t shared_lim, int32_t xdiv, void * out, uint32_t otype, int gateup,
                               void * stream, tqmoe_error * err, const char * what, Glu glu) {
    if (int32_t rc = check_bank(b0, what, err)) return rc;
    if (b1) {
        if (int32_t rc = check_bank(b1, what, err)) return rc;
        if (b1->type != b0->type || b1->rows != b0->rows || b1->cols != b0->cols || b1->experts != b0->experts)
            return fail(err, TQMOE_E_ARG, "%s: the two banks differ in format or shape", what);
    }
    if (!x || !counts || !offsets || !perm || !out || n <= 0 || topk <= 0 || slots < topk) return fail(err, TQMOE_E_ARG, "%s: invalid shape or pointer", what);
    if (!is_act_type(xtype) || !is_act_type(otype)) return fail(err, TQMOE_E_UNSUPPORTED, "%s: unsupported element type", what);
    const int lim_max = gateup ? b0->rows : b0->cols;
    if (slots > topk && (shared_lim <= 0 || shared_lim > lim_max || shared_lim % 32)) return fail(err, TQMOE_E_ARG, "%s: shared_lim must be a multiple of 32 within the bank", what);
    if (b0->experts > 4096) return fail(err, TQMOE_E_ARG, "%s: more than 4096 experts", what);
    if (int32_t rc = need_device(err, what)) return rc;
    const int shared_expert = slots > topk ? b0->experts - 1 : -1;
    if (enqueue_gemm_f16(*b0, b1, x, xtype, counts, offsets, perm, b0->experts, int64_t(n) * slots, xdiv, out, otype, gateup, shared_expert,
                         shared_lim, static_cast<hipStream_t>(stream), glu))
        return fail(err, TQMOE_E_ARG, "%s: too many assignments for one call", what);
    return launched(err, what);
}

extern "C" int32_t tqmoe_expert_gemm_gateup(const tqmoe_bank * gate, const tqmoe_bank * up, const void * x, uint32_t xtype, const int32_t * counts,
                                            const int32_t * offsets, const int32_t * perm, int32_t n, int32_t slots, int32_t topk, int32_t shared_lim, void * act_f16,
                                            void * stream, tqmoe_error * err) {
    if (!up) return fail(err, TQMOE_E_ARG, "tqmoe_expert_gemm_gateup: second bank missing");
    return gemm_f16_common(gate, up, x, xtype, counts, offsets, perm, n, slots, topk, shared_lim, slots, act_f16, TQMOE_F16, 1, stream, err, "tqmoe_expert_gemm_gateup");
}

extern "C" int32_t tqmoe_expert_gemm(const tqmoe_bank * bank, const void * x, uint32_t xtype, const int32_t * counts, const int32_t * offsets, const int32_t * perm,
                                     int32_t n, int32_t slots, int32_t topk, int32_t shared_lim, int32_t per_expert_input, void * y, uint32_t ytype, void * stream,
                                     tqmoe_error * err) {
    return gemm_f16_common(bank, nullptr, x, xtype, counts, offsets, perm, n, slots, topk, shared_lim, per_expert_input ? 1 : slots, y, ytype, 0, stream, err,
                           "tqmoe_expert_gemm");
}

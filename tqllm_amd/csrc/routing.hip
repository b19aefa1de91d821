// Router logits, softmax + top-k, and the stable token-to-expert dispatch.
#include "common.cuh"

namespace tqmoe {
namespace {

// ----------------------------------------------------------------------------------------------------- router
// One wave per router row, kTok tokens per pass; each lane owns 8-element chunks lane, lane + 64, ... of the row.
// Sums in fp32; the order (chunks ascending per lane, then a butterfly over lanes) differs from a column-order host
// sum by ordinary fp32 rounding only.
constexpr int kRouterTok = 4;
template <int WT, int XT>
__global__ __launch_bounds__(256) void router_k(const void * __restrict__ w, const void * __restrict__ shared,
                                                const void * __restrict__ x, float * __restrict__ logits, int h, int e, int n) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int row = blockIdx.x * 4 + wave;  // 0..e (e = the shared gate)
    const int t0 = blockIdx.y * kRouterTok;
    if (row > e) return;                     // whole waves leave together: reductions below see full waves
    const bool has_row = row < e || shared != nullptr;
    const void * wr = row < e ? w : shared;
    const int64_t wbase = row < e ? int64_t(row) * h : 0;
    float acc[kRouterTok];
#pragma unroll
    for (int i = 0; i < kRouterTok; ++i) acc[i] = 0.f;
    if (has_row)
        for (int c = lane * 8; c < h; c += 512) {
            float wv[8];
            load8<WT>(wr, wbase + c, wv);
#pragma unroll
            for (int i = 0; i < kRouterTok; ++i) {
                if (t0 + i < n) {
                    float xv[8];
                    load8<XT>(x, int64_t(t0 + i) * h + c, xv);
#pragma unroll
                    for (int j = 0; j < 8; ++j) acc[i] = fmaf(wv[j], xv[j], acc[i]);
                }
            }
        }
#pragma unroll
    for (int i = 0; i < kRouterTok; ++i) {
        const float s = group_sum<64>(acc[i]);
        if (lane == 0 && t0 + i < n) logits[int64_t(t0 + i) * (e + 1) + row] = s;
    }
}

template <int WT> int32_t launch_router_x(uint32_t xtype, const void * w, const void * sg, const void * x, float * logits,
                                          int h, int e, int n, hipStream_t s) {
    const dim3 grid(unsigned((e + 1 + 3) / 4), unsigned((n + kRouterTok - 1) / kRouterTok));
    switch (xtype) {
        case TQMOE_F32: router_k<WT, TQMOE_F32><<<grid, 256, 0, s>>>(w, sg, x, logits, h, e, n); return 0;
        case TQMOE_F16: router_k<WT, TQMOE_F16><<<grid, 256, 0, s>>>(w, sg, x, logits, h, e, n); return 0;
        case TQMOE_BF16: router_k<WT, TQMOE_BF16><<<grid, 256, 0, s>>>(w, sg, x, logits, h, e, n); return 0;
    }
    return -1;
}

// ------------------------------------------------------------------------------------------------------ top-k
// One wave per token. Probabilities live in LDS (experts floats); lane l owns entries l, l + 64, ...
// Selection rule of the reference: larger probability first, equal probabilities to the lower index.
struct Best { float v; int i; };
__device__ __forceinline__ Best better(Best a, Best b) { return (b.v > a.v || (b.v == a.v && b.i < a.i)) ? b : a; }
__device__ __forceinline__ Best wave_best(Best b) {
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        Best o;
        o.v = __shfl_xor(b.v, d, 64);
        o.i = __shfl_xor(b.i, d, 64);
        b = better(b, o);
    }
    return b;
}

__global__ __launch_bounds__(64) void topk_k(const float * __restrict__ logits, int * __restrict__ ids, float * __restrict__ weights,
                                             float * __restrict__ shared_weights, int e, int k, float scale) {
    extern __shared__ float probs[];
    const int token = blockIdx.x, lane = threadIdx.x;
    const float * x = logits + int64_t(token) * (e + 1);
    float m = -INFINITY;
    for (int j = lane; j < e; j += 64) m = fmaxf(m, x[j]);
    m = wave_max(m);
    float sum = 0.f;
    for (int j = lane; j < e; j += 64) { const float p = expf(x[j] - m); probs[j] = p; sum += p; }
    sum = group_sum<64>(sum);
    for (int j = lane; j < e; j += 64) probs[j] = probs[j] / sum;
    __syncthreads();
    float selected = 0.f;
    for (int s = 0; s < k; ++s) {
        Best b{-INFINITY, e};
        for (int j = lane; j < e; j += 64) b = better(b, Best{probs[j], j});
        b = wave_best(b);
        if (lane == 0) { ids[int64_t(token) * k + s] = b.i; weights[int64_t(token) * k + s] = b.v; }
        selected += b.v;                       // slot order, as the host sums the selected weights
        if ((b.i & 63) == lane) probs[b.i] = -1.f;
    }
    if (lane == 0) {
        const float total = fmaxf(selected, 6.103515625e-5f);
        for (int s = 0; s < k; ++s) {
            float v = weights[int64_t(token) * k + s] / total;
            if (scale != 0.f && scale != 1.f) v *= scale;
            weights[int64_t(token) * k + s] = v;
        }
        if (shared_weights) shared_weights[token] = 1.f / (1.f + expf(-x[e]));
    }
}

// --------------------------------------------------------------------------------------------------- dispatch
// Stable counting sort of the assignments by expert. Chunks of kChunk consecutive assignments; pass 1 counts each
// chunk's experts in LDS, pass 2 turns the per-chunk counts into exclusive prefixes (and counts / offsets), pass 3
// places every assignment at offsets[e] + prefix[chunk][e] + its rank among the chunk's earlier assignments of the
// same expert. Ranks come from ballots (lower lanes of the same expert) and a per-expert running count in LDS that
// waves add to in wave order, so no ordering is left to atomics. A single chunk runs all three passes in one block.
constexpr int kChunk = 1024;

__device__ __forceinline__ void zero_lds(int * a, int n) {
    for (int j = threadIdx.x; j < n; j += blockDim.x) a[j] = 0;
}

// exclusive scan over e of run[0..E) into out[0..E], out[E] = total; one block, E <= 4096, scratch >= blockDim ints
__device__ void block_exclusive_scan(const int * run, int * out, int E, int * scratch) {
    const int tid = threadIdx.x, nt = blockDim.x;
    const int per = (E + nt - 1) / nt, lo = min(tid * per, E), hi = min(lo + per, E);
    int s = 0;
    for (int j = lo; j < hi; ++j) s += run[j];
    scratch[tid] = s;
    __syncthreads();
    for (int d = 1; d < nt; d <<= 1) {  // Hillis-Steele inclusive scan of the per-thread sums
        const int v = tid >= d ? scratch[tid - d] : 0;
        __syncthreads();
        scratch[tid] += v;
        __syncthreads();
    }
    int base = tid ? scratch[tid - 1] : 0;
    for (int j = lo; j < hi; ++j) { out[j] = base; base += run[j]; }
    if (tid == nt - 1) out[E] = scratch[nt - 1];
    __syncthreads();
}

__global__ __launch_bounds__(256) void dispatch_count_k(const int * __restrict__ ids, int * __restrict__ chunk_counts, int A, int E) {
    extern __shared__ int hist[];
    zero_lds(hist, E);
    __syncthreads();
    const int base = blockIdx.x * kChunk;
    for (int i = threadIdx.x; i < kChunk; i += 256) {
        const int a = base + i;
        if (a < A) { const int e = ids[a]; if (e >= 0 && e < E) atomicAdd(&hist[e], 1); }
    }
    __syncthreads();
    for (int j = threadIdx.x; j < E; j += 256) chunk_counts[int64_t(blockIdx.x) * E + j] = hist[j];
}

__global__ __launch_bounds__(1024) void dispatch_scan_k(int * __restrict__ chunk_counts, int * __restrict__ counts,
                                                       int * __restrict__ offsets, int chunks, int E) {
    extern __shared__ int sm[];  // E totals, then 1024 scratch
    for (int e = threadIdx.x; e < E; e += blockDim.x) {
        int run = 0;
        for (int b = 0; b < chunks; ++b) {
            const int v = chunk_counts[int64_t(b) * E + e];
            chunk_counts[int64_t(b) * E + e] = run;
            run += v;
        }
        sm[e] = run;
        counts[e] = run;
    }
    __syncthreads();
    block_exclusive_scan(sm, offsets, E, sm + E);
}

// places one chunk; run[] = per-expert running count inside the chunk (LDS, zeroed by the caller)
__device__ void place_chunk(const int * __restrict__ ids, const int * __restrict__ offsets, const int * __restrict__ prefix,
                            int * __restrict__ perm, int * __restrict__ groups, int capacity, int base, int A, int E, int * run) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
    for (int i0 = 0; i0 < kChunk && base + i0 < A; i0 += blockDim.x) {
        const int a = base + i0 + threadIdx.x;
        int e = a < A ? ids[a] : -1;
        if (e >= E) e = -1;
        // rank of this lane among the wave's earlier lanes of the same expert, and the size of its group
        int rank = 0, size = 0;
        bool last = false;
        unsigned long long todo = __ballot(e >= 0);
        while (todo) {
            const int leader = __ffsll(todo) - 1;
            const int v = __shfl(e, leader, 64);
            const unsigned long long same = __ballot(e == v);
            if (e == v) {
                rank = __popcll(same & ((1ull << lane) - 1ull));
                size = __popcll(same);
                last = (63 - __clzll(same)) == lane;
            }
            todo &= ~same;
        }
        for (int w = 0; w < waves; ++w) {  // waves take their turn in index order
            if (wave == w && e >= 0) {
                const int slot = (prefix ? prefix[e] : 0) + run[e] + rank;
                perm[offsets[e] + slot] = a;
                if (groups && slot < capacity) groups[int64_t(e) * capacity + slot] = a;
            }
            __syncthreads();
            if (wave == w && e >= 0 && last) run[e] += size;
            __syncthreads();
        }
    }
}

__global__ __launch_bounds__(256) void dispatch_place_k(const int * __restrict__ ids, const int * __restrict__ offsets,
                                                        const int * __restrict__ chunk_prefix, int * __restrict__ perm,
                                                        int * __restrict__ groups, int capacity, int A, int E) {
    extern __shared__ int run[];
    zero_lds(run, E);
    __syncthreads();
    place_chunk(ids, offsets, chunk_prefix + int64_t(blockIdx.x) * E, perm, groups, capacity, blockIdx.x * kChunk, A, E, run);
}

// A <= kChunk: everything in one block
__global__ __launch_bounds__(256) void dispatch_small_k(const int * __restrict__ ids, int * __restrict__ counts, int * __restrict__ offsets,
                                                        int * __restrict__ perm, int * __restrict__ groups, int capacity, int A, int E) {
    extern __shared__ int sm[];  // hist E, offs E + 1, scratch 256
    int * hist = sm, * offs = sm + E, * scratch = sm + 2 * E + 1;
    zero_lds(hist, E);
    __syncthreads();
    for (int a = threadIdx.x; a < A; a += 256) { const int e = ids[a]; if (e >= 0 && e < E) atomicAdd(&hist[e], 1); }
    __syncthreads();
    block_exclusive_scan(hist, offs, E, scratch);
    for (int j = threadIdx.x; j < E; j += 256) { counts[j] = hist[j]; offsets[j] = offs[j]; }
    if (threadIdx.x == 0) offsets[E] = offs[E];
    __syncthreads();
    zero_lds(hist, E);
    __syncthreads();
    place_chunk(ids, offs, nullptr, perm, groups, capacity, 0, A, E, hist);
}

}  // namespace
}  // namespace tqmoe

using namespace tqmoe;

extern "C" uint32_t tqmoe_abi_version(void) { return TQMOE_ABI_VERSION; }

extern "C" int32_t tqmoe_router(const void * router, uint32_t wtype, const void * shared_gate, const void * x, uint32_t xtype,
                                float * logits, int32_t hidden, int32_t experts, int32_t n, void * stream, tqmoe_error * err) {
    if (!router || !x || !logits || hidden <= 0 || experts <= 0 || n <= 0) return fail(err, TQMOE_E_ARG, "tqmoe_router: invalid shape or pointer");
    if (hidden % 8) return fail(err, TQMOE_E_ARG, "tqmoe_router: hidden must be a multiple of 8");
    if ((wtype != TQMOE_F32 && wtype != TQMOE_BF16) || !is_act_type(xtype)) return fail(err, TQMOE_E_UNSUPPORTED, "tqmoe_router: unsupported element type");
    if ((n + kRouterTok - 1) / kRouterTok > 65535) return fail(err, TQMOE_E_ARG, "tqmoe_router: too many tokens for one call");
    if (int32_t rc = need_device(err, "tqmoe_router")) return rc;
    const hipStream_t s = static_cast<hipStream_t>(stream);
    if (wtype == TQMOE_F32) launch_router_x<TQMOE_F32>(xtype, router, shared_gate, x, logits, hidden, experts, n, s);
    else launch_router_x<TQMOE_BF16>(xtype, router, shared_gate, x, logits, hidden, experts, n, s);
    return launched(err, "tqmoe_router");
}

extern "C" int32_t tqmoe_topk(const float * logits, int32_t * ids, float * weights, float * shared_weights, int32_t experts,
                              int32_t topk, int32_t n, float scale, void * stream, tqmoe_error * err) {
    if (!logits || !ids || !weights || experts <= 0 || experts > 4096 || topk <= 0 || topk > experts || n <= 0)
        return fail(err, TQMOE_E_ARG, "tqmoe_topk: invalid shape or pointer");
    if (int32_t rc = need_device(err, "tqmoe_topk")) return rc;
    topk_k<<<unsigned(n), 64, size_t(experts) * sizeof(float), static_cast<hipStream_t>(stream)>>>(logits, ids, weights, shared_weights,
                                                                                                  experts, topk, scale);
    return launched(err, "tqmoe_topk");
}

extern "C" size_t tqmoe_dispatch_workspace_bytes(int32_t experts, int32_t n, int32_t topk) {
    if (experts <= 0 || n <= 0 || topk <= 0) return 0;
    const int64_t A = int64_t(n) * topk, chunks = (A + kChunk - 1) / kChunk;
    return chunks <= 1 ? 16 : size_t(chunks) * size_t(experts) * sizeof(int);
}

extern "C" int32_t tqmoe_dispatch(const int32_t * ids, int32_t * counts, int32_t * offsets, int32_t * perm, int32_t * groups,
                                  int32_t capacity, int32_t experts, int32_t n, int32_t topk, void * workspace, size_t workspace_bytes,
                                  void * stream, tqmoe_error * err) {
    if (!ids || !counts || !offsets || !perm || experts <= 0 || experts > 4096 || n <= 0 || topk <= 0 || (groups && capacity <= 0))
        return fail(err, TQMOE_E_ARG, "tqmoe_dispatch: invalid shape or pointer");
    const int64_t A64 = int64_t(n) * topk;
    if (A64 > (1 << 30)) return fail(err, TQMOE_E_ARG, "tqmoe_dispatch: too many assignments");
    const int A = int(A64), chunks = (A + kChunk - 1) / kChunk;
    if (int32_t rc = need_device(err, "tqmoe_dispatch")) return rc;
    const hipStream_t s = static_cast<hipStream_t>(stream);
    if (chunks == 1) {
        dispatch_small_k<<<1, 256, size_t(2 * experts + 1 + 256) * sizeof(int), s>>>(ids, counts, offsets, perm, groups, capacity, A, experts);
        return launched(err, "tqmoe_dispatch");
    }
    if (!workspace || workspace_bytes < tqmoe_dispatch_workspace_bytes(experts, n, topk))
        return fail(err, TQMOE_E_WORKSPACE, "tqmoe_dispatch: workspace of %zu bytes needed", tqmoe_dispatch_workspace_bytes(experts, n, topk));
    int * cc = static_cast<int *>(workspace);
    dispatch_count_k<<<unsigned(chunks), 256, size_t(experts) * sizeof(int), s>>>(ids, cc, A, experts);
    dispatch_scan_k<<<1, 1024, size_t(experts + 1024) * sizeof(int), s>>>(cc, counts, offsets, chunks, experts);
    dispatch_place_k<<<unsigned(chunks), 256, size_t(experts) * sizeof(int), s>>>(ids, offsets, cc, perm, groups, capacity, A, experts);
    return launched(err, "tqmoe_dispatch");
}

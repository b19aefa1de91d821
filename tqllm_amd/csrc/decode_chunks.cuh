// The input rows a decode block serves: assignments that share an expert are cut into chunks, so that a chunk's block
// reads (and decodes) the expert's weights once for all of the chunk's rows.
#pragma once
#include "common.cuh"

namespace tqmoe {

constexpr int kChunkRowsMax = 4;   // input rows per block at most
constexpr int kMaxList = 2048;     // assignments one block can scan (the launchers never pass more in mode 1)
constexpr int kChunkListInts = 2 * kMaxList;   // LDS ints the two functions below work in: the match list, then the copy of the ids

// mode 1: the block's copy of the ids, and its own expert from that copy (one trip to memory for both)
__device__ __forceinline__ int fetch_ids(const int * __restrict__ ids, int A, int a, int mode, int * list) {
    if (mode == 0) return ids[a];
    int * copy = list + kMaxList;
    for (int i = threadIdx.x; i < A; i += blockDim.x) copy[i] = ids[i];
    __syncthreads();
    return copy[a];
}
// mode 0: the block's own assignment only. mode 1: the assignments of ids[0..A) with this block's expert, in index
// order, are cut into chunks of `tp` (at most kChunkRowsMax); the block of each chunk's first assignment serves the chunk
// (returns its size and the assignment indices in tok, -1 past the end) and the other blocks leave (returns 0).
__device__ __forceinline__ int chunk_up(int A, int a, int e, int mode, int tp, int * list, int * meta, int (&tok)[kChunkRowsMax]) {
#pragma unroll
    for (int j = 0; j < kChunkRowsMax; ++j) tok[j] = -1;
    if (mode == 0) { tok[0] = a; return 1; }
    const int * copy = list + kMaxList;      // the ids, fetched by the whole block in one round trip (fetch_ids)
    if (threadIdx.x < 64) {   // one wave walks the ids in order: ballots keep the matches ordered
        const int lane = threadIdx.x;
        int base = 0;
        for (int i0 = 0; i0 < A; i0 += 64) {
            const int i = i0 + lane;
            const bool match = i < A && copy[i] == e;
            const unsigned long long mask = __ballot(match);
            if (match) {
                const int r = base + __popcll(mask & ((1ull << lane) - 1ull));
                if (r < kMaxList) list[r] = i;
                if (i == a) meta[1] = r;
            }
            base += __popcll(mask);
        }
        if (lane == 0) meta[0] = min(base, kMaxList);
    }
    __syncthreads();
    const int cnt = meta[0], rank = meta[1];
    if (rank % tp) return 0;
    const int n = min(tp, cnt - rank);
#pragma unroll
    for (int j = 0; j < kChunkRowsMax; ++j) if (j < n) tok[j] = list[rank + j];
    return n;
}

}  // namespace tqmoe

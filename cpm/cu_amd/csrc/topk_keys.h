// 64-bit ranking keys and the k-round workgroup selection shared by the top-k kernels and the
// draft-tree kernels.
//
// Ordering contract of the reference's bitonic TopK (src/model/topk.cuh:17): value descending,
// equal values -> lower index first.  Every element becomes one key
//   (order-preserving 16-bit image of the fp16 value) << 32 | (0xFFFFFFFF - index)
// so "largest key first" IS that ordering and keys are unique.  Key 0 is an empty slot.
#pragma once
#include "common.h"

namespace cpmcu {

constexpr int kTopkThreads = 256;
constexpr int kChunk = 2048;  // elements per workgroup in the first stage (8 per thread)
constexpr int kPerThread = 8;
constexpr int kMaxCand = kTopkThreads * kPerThread;  // candidates the merge stage can hold

__device__ inline uint32_t ord16(uint16_t b) {
    if (b == 0x8000u) b = 0;  // -0 == +0 for the comparator
    return (b & 0x8000u) ? (uint32_t)(~b & 0xFFFFu) : (uint32_t)(b | 0x8000u);
}
__device__ inline uint64_t make_key(uint16_t bits, int idx) {
    return ((uint64_t)ord16(bits) << 32) | (uint32_t)(0xFFFFFFFFu - (uint32_t)idx);
}
__device__ inline uint16_t key_bits(uint64_t key) {
    const uint32_t o = (uint32_t)(key >> 32);
    return (o & 0x8000u) ? (uint16_t)(o & 0x7FFFu) : (uint16_t)(~o & 0xFFFFu);
}
__device__ inline int key_index(uint64_t key) { return (int)(0xFFFFFFFFu - (uint32_t)key); }

__device__ inline uint64_t wave_max_u64(uint64_t v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const uint32_t lo = __shfl_xor((uint32_t)v, off);
        const uint32_t hi = __shfl_xor((uint32_t)(v >> 32), off);
        const uint64_t o = ((uint64_t)hi << 32) | lo;
        v = o > v ? o : v;
    }
    return v;
}

// k rounds of workgroup-wide max over the keys held in registers; round j's winner goes to
// emit(j, key), called by thread 0.  Keys equal to 0 are empty slots.  One barrier per round: the
// per-wave maxima alternate between two LDS buffers, so a wave that runs ahead into the next round
// writes the other buffer (it cannot get two rounds ahead: the barrier in between needs every wave).
// Ends with a barrier, so whatever emit stored in LDS is visible to the workgroup afterwards.
template <typename Emit>
__device__ inline void select_topk(uint64_t (&keys)[kPerThread], int top, Emit emit) {
    __shared__ uint64_t wave_best[2][kTopkThreads / 64];
    const int wave = threadIdx.x >> 6;
    const int lane = threadIdx.x & 63;
    for (int round = 0; round < top; ++round) {
        uint64_t mine = 0;
#pragma unroll
        for (int e = 0; e < kPerThread; ++e) mine = keys[e] > mine ? keys[e] : mine;
        const uint64_t wbest = wave_max_u64(mine);
        uint64_t* wb = wave_best[round & 1];
        if (lane == 0) wb[wave] = wbest;
        __syncthreads();
        uint64_t best = wb[0];
#pragma unroll
        for (int w = 1; w < kTopkThreads / 64; ++w) best = wb[w] > best ? wb[w] : best;
        if (best != 0 && mine == best) {
#pragma unroll
            for (int e = 0; e < kPerThread; ++e)
                if (keys[e] == best) keys[e] = 0;
        }
        if (threadIdx.x == 0) emit(round, best);
    }
    __syncthreads();
}

}  // namespace cpmcu

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

// Wave-wide reductions on the DPP data path (no LDS round trip per step).  Each of the four steps
// exchanges with the lane at xor 1, xor 2, then the mirror lane of its group of 8 and of its row of
// 16 -- after the earlier steps the groups are uniform, so a mirror is as good as an xor -- and the
// four row results are combined through scalar registers.  Every lane gets the result.
template <int CTRL>
__device__ inline uint32_t dpp_mov(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xF, 0xF, true);
}
constexpr int kDppXor1 = 0xB1, kDppXor2 = 0x4E, kDppHalfMirror = 0x141, kDppMirror = 0x140;

template <typename Op>
__device__ inline uint32_t wave_reduce_b32(uint32_t v, Op op) {
    v = op(v, dpp_mov<kDppXor1>(v));
    v = op(v, dpp_mov<kDppXor2>(v));
    v = op(v, dpp_mov<kDppHalfMirror>(v));
    v = op(v, dpp_mov<kDppMirror>(v));
    const uint32_t r0 = __builtin_amdgcn_readlane(v, 0), r1 = __builtin_amdgcn_readlane(v, 16);
    const uint32_t r2 = __builtin_amdgcn_readlane(v, 32), r3 = __builtin_amdgcn_readlane(v, 48);
    return op(op(r0, r1), op(r2, r3));
}
__device__ inline float wave_max_f32(float v) {
    return __builtin_bit_cast(float, wave_reduce_b32(__builtin_bit_cast(uint32_t, v), [](uint32_t a, uint32_t b) {
        return __builtin_bit_cast(uint32_t, fmaxf(__builtin_bit_cast(float, a), __builtin_bit_cast(float, b)));
    }));
}
__device__ inline float wave_sum_f32(float v) {
    return __builtin_bit_cast(float, wave_reduce_b32(__builtin_bit_cast(uint32_t, v), [](uint32_t a, uint32_t b) {
        return __builtin_bit_cast(uint32_t, __builtin_bit_cast(float, a) + __builtin_bit_cast(float, b));
    }));
}

__device__ inline uint64_t wave_max_u64(uint64_t v) {
    const auto step = [](uint64_t a, uint32_t lo, uint32_t hi) {
        const uint64_t o = ((uint64_t)hi << 32) | lo;
        return o > a ? o : a;
    };
    v = step(v, dpp_mov<kDppXor1>((uint32_t)v), dpp_mov<kDppXor1>((uint32_t)(v >> 32)));
    v = step(v, dpp_mov<kDppXor2>((uint32_t)v), dpp_mov<kDppXor2>((uint32_t)(v >> 32)));
    v = step(v, dpp_mov<kDppHalfMirror>((uint32_t)v), dpp_mov<kDppHalfMirror>((uint32_t)(v >> 32)));
    v = step(v, dpp_mov<kDppMirror>((uint32_t)v), dpp_mov<kDppMirror>((uint32_t)(v >> 32)));
    uint64_t best = 0;
#pragma unroll
    for (int r = 0; r < 64; r += 16) {
        const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(v >> 32), r);
        const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)v, r);
        const uint64_t o = ((uint64_t)hi << 32) | lo;
        best = o > best ? o : best;
    }
    return best;
}

// The fused log-softmax ranks f16((z - max) - ln sum) (src/model/eagle.cuh:87), a monotone map of z that merges
// neighbours.  Given the ordered 16-bit image `bound` of a z that has at least k elements at or above it, this is the
// lowest image whose z can still map to the mapped bound's value or above: four ulps of the mapped bound below it, one
// step more for the rounding of that difference and one for -0.  0: no usable bound (every element is a candidate).
template <typename E>
__device__ inline uint32_t mapped_lower_image(uint32_t bound, float m, float lse) {
    if (bound == 0) return 0;
    const uint16_t zb = (uint16_t)((bound & 0x8000u) ? (bound ^ 0x8000u) : (bound ^ 0xFFFFu));
    const float zl = Elem<E>::from_bits(zb);
    const uint16_t y = Elem<E>::to_bits((zl - m) - lse);
    constexpr int kM = Elem<E>::kMantissaBits, kBias = Elem<E>::kExponentBias, kEmax = (1 << Elem<E>::kExponentBits) - 1;
    const int e = (y >> kM) & kEmax;
    const int e4 = (e ? e - kBias - kM : 1 - kBias - kM) + 2;  // exponent of four ulps of the mapped bound
    const float zlo = zl - (e4 >= -126 ? __uint_as_float((uint32_t)(e4 + 127) << 23) : ldexpf(1.f, e4));
    if (e != kEmax && zlo == zlo && fabsf(zlo) <= Elem<E>::kMaxFinite) {  // finite mapped bound, representable lower bound
        const uint16_t lb = Elem<E>::to_bits(zlo);
        const uint32_t o = (uint32_t)(lb ^ ((lb & 0x8000u) ? 0xFFFFu : 0x8000u));
        return o > 2 ? o - 2 : 0;
    }
    return 0;
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

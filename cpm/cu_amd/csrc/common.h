// Shared host/device helpers of libcpmcu_amd (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <cstdarg>
#include <cstdio>
#include <string>

#include "../../../include/cpmcu_amd.h"

namespace cpmcu {

typedef _Float16 f16;
typedef f16 f16x2 __attribute__((ext_vector_type(2)));
typedef f16 f16x4 __attribute__((ext_vector_type(4)));
typedef f16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

// bfloat16, the second element type of the path (src/entry.cu:26-59: torch_dtype 0 = half, 1 = bfloat16).  Every kernel that
// does arithmetic on 16-bit values is a template on the element type E; Elem<E> names its vectors and the few operations
// that differ: the MFMA that takes it, the conversions, the two-way dot product.  Kernels that only move values
// (append, compaction, gathers, the weight tiling) work on 16-bit patterns and serve both.
typedef __bf16 bf16;
typedef bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef bf16 bf16x8 __attribute__((ext_vector_type(8)));

template <typename E>
struct Elem;
template <>
struct Elem<f16> {
    typedef f16x2 x2;
    typedef f16x4 x4;
    typedef f16x8 x8;
    static constexpr int kDtype = 0;
    __device__ static inline f32x16 mfma_32x32x16(x8 a, x8 b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0); }
    __device__ static inline f32x4 mfma_16x16x32(x8 a, x8 b, f32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0); }
    __device__ static inline float dot2_acc(x2 a, x2 b, float c) { return __builtin_amdgcn_fdot2(a, b, c, false); }
    __device__ static inline float from_bits(uint16_t h) { return (float)__builtin_bit_cast(f16, h); }
    __device__ static inline uint16_t to_bits(float f) { return __builtin_bit_cast(uint16_t, (f16)f); }
    static constexpr int kMantissaBits = 10, kExponentBits = 5, kExponentBias = 15;
    static constexpr float kMaxFinite = 65504.f;
};
template <>
struct Elem<bf16> {
    typedef bf16x2 x2;
    typedef bf16x4 x4;
    typedef bf16x8 x8;
    static constexpr int kDtype = 1;
    __device__ static inline f32x16 mfma_32x32x16(x8 a, x8 b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }
    __device__ static inline f32x4 mfma_16x16x32(x8 a, x8 b, f32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0); }
    __device__ static inline float dot2_acc(x2 a, x2 b, float c) { return __builtin_amdgcn_fdot2_f32_bf16(a, b, c, false); }
    __device__ static inline float from_bits(uint16_t h) { return __uint_as_float((uint32_t)h << 16); }
    __device__ static inline uint16_t to_bits(float f) { return __builtin_bit_cast(uint16_t, (bf16)f); }
    static constexpr int kMantissaBits = 7, kExponentBits = 8, kExponentBias = 127;
    static constexpr float kMaxFinite = 3.3895313892515355e38f;
};

constexpr int kPage = CPMCU_PAGE_SIZE;    // tokens per KV page
constexpr int kHeadDim = CPMCU_HEAD_DIM;  // the only head_dim the kernels are built for
constexpr int kMaxTree = CPMCU_MAX_TREE;

// Slot of token t inside its aligned group of 16 in the transposed V pages:
// bits 2 and 3 of the token index are swapped (an involution).
__host__ __device__ inline int v_slot16(int t) { return (t & ~12) | ((t & 4) << 1) | ((t & 8) >> 1); }

// ---- error plumbing (thread-local message, integer status) ----
void set_error(const char* fmt, ...);
hipStream_t resolve_stream(void* stream);  // NULL -> the library's blocking stream

#define CPMCU_CHECK_ARG(cond, ...)                 \
    do {                                           \
        if (!(cond)) {                             \
            ::cpmcu::set_error(__VA_ARGS__);       \
            return CPMCU_ERR_INVALID_ARGUMENT;     \
        }                                          \
    } while (0)

#define CPMCU_HIP(expr)                                                                          \
    do {                                                                                         \
        hipError_t e__ = (expr);                                                                 \
        if (e__ != hipSuccess) {                                                                 \
            ::cpmcu::set_error("%s failed: %s (%s:%d)", #expr, hipGetErrorString(e__), __FILE__, \
                               __LINE__);                                                        \
            return CPMCU_ERR_HIP;                                                                \
        }                                                                                        \
    } while (0)

#define CPMCU_LAUNCH_CHECK() CPMCU_HIP(hipGetLastError())

inline int ceil_div(int a, int b) { return (a + b - 1) / b; }
inline size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

}  // namespace cpmcu

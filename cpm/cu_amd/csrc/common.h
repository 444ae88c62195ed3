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

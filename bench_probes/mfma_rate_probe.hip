// Measurement helper for gfx950 (MI355X): what the matrix pipes deliver to a kernel that does nothing
// else.  The roofline fraction of the attention kernel is quoted against the published peak
// (2.5 PFLOP/s dense fp16 MFMA); this probe says how much of it a register-resident MFMA loop reaches on
// the same GPU as a function of the operand DATA, because the rate the chip sustains depends on how
// many bits toggle (clocks follow the power drawn).  No counterpart in the reference, and not part of
// libcpmcu_amd: bench.py loads this file's own small shared library (bench_probes/libbench_probes.so).
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace {

typedef _Float16 f16;
typedef f16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int kProbeThreads = 512;  // 8 waves, two per SIMD
constexpr int kProbeOperands = 16;  // 8 A and 8 B operand registers (of 8 halves) per lane

// Every lane keeps 8 A and 8 B operands in registers and issues `iters` x 16 MFMAs on four independent
// accumulator chains, cycling through the operands so that consecutive MFMAs see different data.
__global__ __launch_bounds__(kProbeThreads, 1) void mfma_rate_probe_kernel(const f16x8* __restrict__ operands, int iters,
                                                                           float* __restrict__ out) {
    const int tid = threadIdx.x;
    f16x8 a[8], b[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        a[i] = operands[i * kProbeThreads + tid];
        b[i] = operands[(8 + i) * kProbeThreads + tid];
    }
    f32x16 acc[4];
#pragma unroll
    for (int c = 0; c < 4; ++c)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[c][r] = 0.f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int x = 0; x < 16; ++x) acc[x % 4] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[x % 8], b[(x * 3) % 8], acc[x % 4], 0, 0, 0);
    }
    float s = 0.f;
#pragma unroll
    for (int c = 0; c < 4; ++c)
#pragma unroll
        for (int r = 0; r < 16; ++r) s += acc[c][r];
    out[(size_t)blockIdx.x * kProbeThreads + tid] = s;
}

}  // namespace

// Bytes of fp16 operand data one launch reads: 16 operand registers of 8 halves for each of 512 threads.
extern "C" size_t bench_mfma_rate_probe_operand_bytes(void) { return (size_t)kProbeOperands * kProbeThreads * sizeof(f16x8); }

// Enqueues `workgroups` workgroups of 8 waves on `stream` (NULL = the null stream), every lane issuing
// iters x 16 v_mfma_f32_32x32x16_f16 on four accumulator chains from operands held in registers.
// out: device float[workgroups * 512].  *flops (host, may be NULL) receives the floating-point
// operations of the launch.  Returns 0, or a HIP error code / -1 for bad arguments.
extern "C" int bench_mfma_rate_probe(const void* operands, int iters, int workgroups, float* out, double* flops, void* stream) {
    if (!operands || !out || iters < 1 || workgroups < 1 || workgroups > 4096) return -1;
    hipLaunchKernelGGL(mfma_rate_probe_kernel, dim3(workgroups), dim3(kProbeThreads), 0, (hipStream_t)stream, (const f16x8*)operands, iters,
                       out);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return (int)e;
    if (flops) *flops = (double)workgroups * (kProbeThreads / 64) * (double)iters * 16.0 * (2.0 * 32 * 32 * 16);
    return 0;
}

// Measurement helper for gfx950 (MI355X): what the matrix pipes deliver to a kernel that does nothing
// else.  The roofline fraction of the attention kernel is quoted against the published peak
// (2.5 PFLOP/s dense fp16 MFMA); this probe says how much of it a register-resident MFMA loop reaches on
// the same GPU as a function of the operand DATA, because the rate the chip sustains depends on how
// many bits toggle (clocks follow the power drawn).  No counterpart in the reference.
#include "common.h"

namespace cpmcu {
namespace {

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
}  // namespace cpmcu

using namespace cpmcu;

extern "C" size_t cpmcu_mfma_rate_probe_operand_bytes(void) { return (size_t)kProbeOperands * kProbeThreads * sizeof(f16x8); }

extern "C" int cpmcu_mfma_rate_probe(const void* operands, int iters, int workgroups, float* out, double* flops, void* stream) {
    CPMCU_CHECK_ARG(operands && out, "mfma_rate_probe: null pointer argument");
    CPMCU_CHECK_ARG(iters >= 1 && workgroups >= 1 && workgroups <= 4096, "mfma_rate_probe: iters=%d, workgroups=%d", iters, workgroups);
    hipLaunchKernelGGL(mfma_rate_probe_kernel, dim3(workgroups), dim3(kProbeThreads), 0, resolve_stream(stream), (const f16x8*)operands, iters,
                       out);
    CPMCU_LAUNCH_CHECK();
    if (flops) *flops = (double)workgroups * (kProbeThreads / 64) * (double)iters * 16.0 * (2.0 * 32 * 32 * 16);
    return CPMCU_OK;
}

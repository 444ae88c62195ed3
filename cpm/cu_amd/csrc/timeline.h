// Wall-clock stamps inside the kernels, for the timelines quoted in the design notes: compiled in only with
// -DCPMCU_TIMELINE (the build script links those objects into a library of their own, libcpmcu_amd_timeline.so, which
// nothing loads but `python -m cpm.cu_amd.timeline`).  Without the define every macro below is empty and the kernels are
// the product's, instruction for instruction.
//   One record of 16 words per workgroup (the first 1024 of a launch): stamps are reads of the 100 MHz wall clock taken
//   by thread 0, notes are plain values.  Kernels that keep their own count of outstanding memory operations take
//   their stamps into registers (CPMCU_CLOCK) and store them at the very end (CPMCU_STAMP_VALUE).
#pragma once
#ifdef CPMCU_TIMELINE
#define CPMCU_TIMELINE_STORAGE(name) __device__ unsigned long long name[1024 * 16];
#define CPMCU_CLOCK_VAR(var) unsigned long long var = 0
#define CPMCU_CLOCK(var) var = wall_clock64()
#define CPMCU_STAMP(buf, wg, slot)                                                  \
    do {                                                                            \
        if (threadIdx.x == 0 && (wg) < 1024) buf[(wg) * 16 + (slot)] = wall_clock64(); \
    } while (0)
#define CPMCU_STAMP_VALUE(buf, wg, slot, value)                                                      \
    do {                                                                                             \
        if (threadIdx.x == 0 && (wg) < 1024) buf[(wg) * 16 + (slot)] = (unsigned long long)(value);  \
    } while (0)
#define CPMCU_TIMELINE_READER(fn, buf)                                                                          \
    extern "C" int fn(void* host_1024x16_u64) {                                                                 \
        if (hipDeviceSynchronize() != hipSuccess) return 1;                                                     \
        if (hipMemcpyFromSymbol(host_1024x16_u64, HIP_SYMBOL(buf), sizeof(buf)) != hipSuccess) return 1;        \
        static const unsigned long long zeros[1024 * 16] = {0};                                                 \
        return hipMemcpyToSymbol(HIP_SYMBOL(buf), zeros, sizeof(zeros)) == hipSuccess ? 0 : 1;                  \
    }
#else
#define CPMCU_TIMELINE_STORAGE(name)
#define CPMCU_CLOCK_VAR(var)
#define CPMCU_CLOCK(var) \
    do {                 \
    } while (0)
#define CPMCU_STAMP(buf, wg, slot) \
    do {                           \
    } while (0)
#define CPMCU_STAMP_VALUE(buf, wg, slot, value) \
    do {                                        \
    } while (0)
#define CPMCU_TIMELINE_READER(fn, buf)
#endif

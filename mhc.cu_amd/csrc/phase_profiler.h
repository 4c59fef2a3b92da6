// In-kernel phase profiler (profile build only: -DMHC_PHASE_PROFILE, libmhc_hip_profile.so).
//
// Counterpart of the reference's DeviceProfiler / HostProfiler (src/csrc/include/utils.cuh:239-389):
// there every block records (SM id, tag, globaltimer start, duration) entries; here wave 0 of a
// workgroup stamps s_memtime (the shader clock) at the phase boundaries of a kernel into a
// fixed table, one row per workgroup, and the host reads the table back after the launch
// (mhc_phase_read).  Differences of consecutive stamps are the phase durations in clock ticks;
// absolute values are only comparable inside one workgroup (the counters of different XCDs are
// not aligned).  In the normal build MHC_PHASE(...) expands to nothing.
#pragma once

#include <hip/hip_runtime.h>

namespace mhc {

constexpr int kPhaseMaxWg = 4096;   // workgroups recorded per kernel (the first ones by linear id)
constexpr int kPhaseMaxMarks = 8;   // stamps per workgroup
enum PhaseKernel { kPhaseFwdFused = 0, kPhaseBwdSlab = 1, kPhaseProjBwd = 2, kPhaseProjFwd = 3, kPhaseGramSmall = 4, kPhaseDxSmall = 5, kPhaseFwdOnepass = 6, kPhaseCoefFwdWide = 7, kPhaseCoefBwdWide = 8, kPhaseColSlab = 9, kPhaseKernels = 10 };

#ifdef MHC_PHASE_PROFILE
extern __device__ unsigned long long g_phase[kPhaseKernels][kPhaseMaxWg][kPhaseMaxMarks];

__device__ __forceinline__ unsigned long long phase_clock() {
    unsigned long long t;
    asm volatile("s_memtime %0\n s_waitcnt lgkmcnt(0)" : "=s"(t)::"memory");
    return t;
}
// stamp slot `mark` of workgroup `wg` (call from every thread: thread 0 writes)
__device__ __forceinline__ void phase_mark(int kernel, int wg, int mark) {
    const unsigned long long t = phase_clock();
    if (threadIdx.x == 0 && wg < kPhaseMaxWg) g_phase[kernel][wg][mark] = t;
}
// add (now - since) to slot `mark`, return now: for phases that repeat inside a loop
__device__ __forceinline__ unsigned long long phase_add(int kernel, int wg, int mark, unsigned long long since) {
    const unsigned long long t = phase_clock();
    if (threadIdx.x == 0 && wg < kPhaseMaxWg) g_phase[kernel][wg][mark] += t - since;
    return t;
}
// the same from a chosen thread of the workgroup (a second timeline, e.g. of another wave)
__device__ __forceinline__ unsigned long long phase_add_by(int thread, int kernel, int wg, int mark, unsigned long long since) {
    const unsigned long long t = phase_clock();
    if ((int)threadIdx.x == thread && wg < kPhaseMaxWg) g_phase[kernel][wg][mark] += t - since;
    return t;
}
#define MHC_PHASE_ADD_BY(thread, kernel, wg, mark, var) var = ::mhc::phase_add_by(thread, kernel, wg, mark, var)
#define MHC_PHASE(kernel, wg, mark) ::mhc::phase_mark(kernel, wg, mark)
#define MHC_PHASE_BEGIN(var) unsigned long long var = ::mhc::phase_clock()
#define MHC_PHASE_ZERO(kernel, wg)                                                        \
    do {                                                                                  \
        if (threadIdx.x < ::mhc::kPhaseMaxMarks && (wg) < ::mhc::kPhaseMaxWg)             \
            ::mhc::g_phase[kernel][wg][threadIdx.x] = 0;                                  \
    } while (0)
#define MHC_PHASE_ADD(kernel, wg, mark, var) var = ::mhc::phase_add(kernel, wg, mark, var)
#else
#define MHC_PHASE(kernel, wg, mark) ((void)0)
#define MHC_PHASE_BEGIN(var) ((void)0)
#define MHC_PHASE_ZERO(kernel, wg) ((void)0)
#define MHC_PHASE_ADD(kernel, wg, mark, var) ((void)0)
#define MHC_PHASE_ADD_BY(thread, kernel, wg, mark, var) ((void)0)
#endif

}  // namespace mhc

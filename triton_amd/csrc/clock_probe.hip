// Shader clock under load.  One wave reads the two hardware time counters - s_memtime, a free-running
// counter on the shader core clock, and s_memrealtime, the constant-rate real-time counter whose rate the
// runtime reports as the wall clock rate - at its start and again after `duration_us` of real time, and
// writes both differences: launched on a second stream next to the kernel under study, their ratio is the
// clock that kernel ran at (the board lowers the clock of MFMA-heavy kernels to stay within its power
// limit, so the nominal clock says nothing about them).  The measurement analogue of the reference's
// clock handling in its peak formulas (python/triton/testing.py:404-426 take the clock as an argument).
#include "common.h"
#include "launch.h"

namespace mi355 {

__global__ void clock_probe_kernel(unsigned long long* out, unsigned long long real_ticks) {
#if MI355_DEVICE_PASS
  if (threadIdx.x != 0) return;
  const unsigned long long r0 = __builtin_amdgcn_s_memrealtime();
  const unsigned long long c0 = __builtin_readcyclecounter();
  unsigned long long r1 = r0;
  // bounded twice: by the real-time counter and by the iteration count (s_sleep 64 = 4096 cycles, about
  // 2 us at any clock this board runs at, so the count alone ends the wave after at most ~10 s)
  for (int i = 0; i < (1 << 22) && r1 - r0 < real_ticks; i++) {
    __builtin_amdgcn_s_sleep(64);
    r1 = __builtin_amdgcn_s_memrealtime();
  }
  const unsigned long long c1 = __builtin_readcyclecounter();
  out[0] = c1 - c0;
  out[1] = r1 - r0;
#endif
}

int clock_probe_launch(unsigned long long* out, unsigned long long real_ticks, hipStream_t stream) {
  hipLaunchKernelGGL(clock_probe_kernel, dim3(1), dim3(64), 0, stream, out, real_ticks);
  return (int)hipGetLastError();
}

}  // namespace mi355

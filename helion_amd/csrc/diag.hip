// Measurement aid (no counterpart in the reference): the engine clock a kernel actually runs at.
// One wave reads the shader-clock counter (s_memtime, counts engine clocks of its XCD) and the constant
// 100 MHz counter (s_memrealtime) at its start, sleeps until `ticks` of the 100 MHz counter have passed and reads
// both again: clock = d(memtime) / d(memrealtime) * 100 MHz.  Launched on a second stream next to a running
// kernel it reports the clock that kernel is being run at (the chip is power-limited: the sustained clock under
// MFMA load is well below the 2.4 GHz maximum).
#include "hx_common.h"

__global__ __launch_bounds__(64) void hx_clock_probe_kernel(uint64_t* __restrict__ out, long long ticks) {
  const uint64_t c0 = __builtin_readcyclecounter();
  const uint64_t r0 = wall_clock64();
  uint64_t r1 = r0;
  // bounded, sparse wait: every iteration sleeps ~8000 clocks (3-4 us) before it reads the 100 MHz counter again, and
  // 64 iterations (about 0.25 ms) end the kernel even if that counter were stuck
  for (int i = 0; i < 64 && (long long)(r1 - r0) < ticks; ++i) {
    __builtin_amdgcn_s_sleep(127);
    r1 = wall_clock64();
  }
  const uint64_t c1 = __builtin_readcyclecounter();
  r1 = wall_clock64();
  if (threadIdx.x == 0) {
    out[0] = c1 - c0;
    out[1] = r1 - r0;
  }
}

extern "C" int hx_clock_probe(uint64_t* out2, int64_t ticks_100mhz, void* stream) {
  if (!out2 || ticks_100mhz <= 0 || ticks_100mhz > 10000) {
    hx_set_error("hx_clock_probe: out2 must be a device pointer to two uint64 and 0 < ticks <= 10000 (100 us)");
    return HX_ERR_BAD_ARG;
  }
  hx_launch(hx_clock_probe_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, out2, (long long)ticks_100mhz);
  const hipError_t e = hx_launch_status();
  if (e != hipSuccess) {
    hx_set_error("hx_clock_probe: launch failed: %s", hipGetErrorString(e));
    return (int)e;
  }
  return 0;
}

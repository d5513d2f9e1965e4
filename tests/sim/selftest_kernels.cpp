// Negative controls for the host execution model itself: small kernels with a deliberate defect each, which the model
// must expose (tests/test_sim_model.py), next to the correct form, which it must pass.  Compiled into the model's
// library only; not part of the product.
#include "hx_common.h"

// mode 0: 1 KB per wave global -> LDS by DMA, wait, barrier, every work-item copies its 16 bytes out: correct.
// mode 1: the same without the wait: the copy reads the LDS while the transfer may still be in flight.
// mode 2: the wait is there but the barrier is not, and a work-item reads what ANOTHER wave fetched.
// mode 3: correct protocol, but the last work-item reads its 16 bytes one element past the end of `in`.
__global__ void hx_sim_selftest_kernel(const uint8_t* in, uint8_t* out, int mode) {
  __shared__ __attribute__((aligned(1024))) uint8_t buf[4 * 1024];
  const int tid = threadIdx.x, w = tid >> 6;
  const uint32_t lds0 = hx_lds_addr(&buf[0]) + w * 1024;
  long off = (long)tid * 16;
  if (mode == 3 && tid == 255) off += 1;
  hx_g2l16_s(in, (uint32_t)off, lds0);
  if (mode != 1) HX_WAIT_VM0();
  if (mode != 2) __syncthreads();
  const int src = mode == 2 ? ((tid + 64) & 255) : tid;  // mode 2: the next wave's data
  const v4i v = *(const v4i*)(&buf[src * 16]);
  *(v4i*)(out + tid * 16) = v;
}

extern "C" int hx_sim_selftest(const void* in, void* out, int mode) {
  hx_launch(hx_sim_selftest_kernel, dim3(1), dim3(256), 0, (hipStream_t) nullptr, (const uint8_t*)in, (uint8_t*)out, mode);
  return (int)hx_launch_status();
}

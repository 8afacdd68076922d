// Element-wise decode of narrow-format codes to fp32 with the same closed forms the kernels
// use (formats.h); lets callers and tests read the decode tables off the device.
#include "common.h"
#include "formats.h"
#include "launch.h"

namespace mi355 {

__global__ void dequant_kernel(const uint8_t* codes, float* out, int64_t n, int fmt) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  uint8_t c = codes[i];
  switch (fmt) {
    case 0: out[i] = e4m3_to_f32(c); break;
    case 1: out[i] = e5m2_to_f32(c); break;
    case 2: out[2 * i] = e2m1_to_f32(c & 15); out[2 * i + 1] = e2m1_to_f32(c >> 4); break;
    default: out[i] = e8m0_to_f32(c); break;
  }
}

int dequant_launch(const uint8_t* codes, float* out, int64_t n, int fmt, hipStream_t stream) {
  int64_t blocks = (n + 255) / 256;
  hipLaunchKernelGGL(dequant_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, codes, out, n, fmt);
  return (int)hipGetLastError();
}

}  // namespace mi355

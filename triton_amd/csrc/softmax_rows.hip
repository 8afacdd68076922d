// Row softmax applied in place to a GEMM result: the DO_SOFTMAX epilogue of the reference's dot
// test (python/test/unit/language/test_core.py:3136-3141: z - max, exp, sum, divide; the reference
// does it inside its single tile, here it is a second launch over the rows of C).
// One wave per row: the row is read twice (max, then exp and sum) and written once, all in fp32
// arithmetic whatever the storage type.
#include "common.h"
#include "launch.h"

namespace mi355 {

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o));
  return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
  return v;
}

__device__ __forceinline__ void store_out(void* c, int64_t off, int dtype, float v) {
  if (dtype == 4) ((float*)c)[off] = v;
  else if (dtype == 1) ((__bf16*)c)[off] = (__bf16)v;
  else ((_Float16*)c)[off] = (_Float16)v;
}

__global__ __launch_bounds__(256) void softmax_rows_kernel(void* C, int M, int N, int64_t scm, int64_t scn, int dtype) {
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= M) return;
  const int64_t base = (int64_t)row * scm;
  float mx = -INFINITY;
  for (int n = lane; n < N; n += 64) mx = fmaxf(mx, load_aux(C, base + (int64_t)n * scn, dtype));
  mx = wave_max(mx);
  float sum = 0.f;
  for (int n = lane; n < N; n += 64) sum += __expf(load_aux(C, base + (int64_t)n * scn, dtype) - mx);
  sum = wave_sum(sum);
  const float inv = 1.f / sum;
  for (int n = lane; n < N; n += 64) {
    const int64_t off = base + (int64_t)n * scn;
    store_out(C, off, dtype, __expf(load_aux(C, off, dtype) - mx) * inv);
  }
}

int softmax_rows_launch(void* C, int M, int N, int64_t scm, int64_t scn, int dtype, hipStream_t stream) {
  softmax_rows_kernel<<<dim3((M + 3) / 4), dim3(256), 0, stream>>>(C, M, N, scm, scn, dtype);
  return (int)hipGetLastError();
}

}  // namespace mi355

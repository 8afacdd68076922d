// Second launch of a split-K product: C = act(alpha * (sum over the splits of the fp32 partial tiles) + addend), one
// rounding to the output type - the epilogue of the reference's kernel (python/tutorials/03-matrix-multiplication.py:
// 304-316) on sums that gemm_splitk_kernel left in the workspace as [splits][M][N] floats.  The slices are added in
// split order, so the result does not depend on how the workgroups of the first launch were scheduled.
#include "common.h"
#include "launch.h"
#include "formats.h"

namespace mi355 {

namespace {

__global__ __launch_bounds__(256) void splitk_reduce_kernel(GemmStridedArgs p, const float* __restrict__ ws, int splits) {
  // a thread per four consecutive columns of a row (one 16-byte load per slice where N is a multiple of 4)
  const int groups = (p.N + 3) / 4;
  const int64_t id = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (id >= (int64_t)p.M * groups) return;
  const int m = (int)(id / groups), n = (int)(id % groups) * 4;
  const int64_t slice = (int64_t)p.M * p.N;
  const float* src = ws + (int64_t)m * p.N + n;
  float v[4] = {0.f, 0.f, 0.f, 0.f};
  if (p.N % 4 == 0) {
    for (int z = 0; z < splits; z++) {
      const f32x4 t = *(const f32x4*)(src + z * slice);
#pragma unroll
      for (int e = 0; e < 4; e++) v[e] += t[e];
    }
  } else {
    for (int z = 0; z < splits; z++)
#pragma unroll
      for (int e = 0; e < 4; e++)
        if (n + e < p.N) v[e] += src[z * slice + e];
  }
  float alpha = 1.f;
  if (p.a_scale) alpha *= *p.a_scale;
  if (p.b_scale) alpha *= *p.b_scale;
#pragma unroll
  for (int e = 0; e < 4; e++) {
    if (n + e >= p.N) break;
    float x = v[e] * alpha;
    if (p.aux) x += load_aux(p.aux, (int64_t)m * p.aux_sm + (int64_t)(n + e) * p.aux_sn, p.aux_dtype);
    if (p.activation == 1) x = x >= 0.f ? x : 0.01f * x;
    const int64_t idx = (int64_t)m * p.scm + (int64_t)(n + e) * p.scn;
    switch (p.out_dtype) {
      case 0: ((_Float16*)p.C)[idx] = (_Float16)x; break;
      case 1: ((__bf16*)p.C)[idx] = (__bf16)x; break;
      case 2: ((uint8_t*)p.C)[idx] = f32_to_e4m3(x); break;
      case 3: ((uint8_t*)p.C)[idx] = f32_to_e5m2(x); break;
      default: ((float*)p.C)[idx] = x; break;
    }
  }
}

}  // namespace

int splitk_reduce_launch(const GemmStridedArgs& out, const float* workspace, int splits, hipStream_t stream) {
  const int64_t threads = (int64_t)out.M * ((out.N + 3) / 4);
  const int64_t blocks = (threads + 255) / 256;
  if (blocks <= 0 || blocks > 0x7fffffffll) return -1;
  hipLaunchKernelGGL(splitk_reduce_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, out, workspace, splits);
  return (int)hipGetLastError();
}

}  // namespace mi355

// Strided GEMM for operands the MFMA kernels do not take (no unit stride, rows not 16-byte
// aligned, K not a multiple of the vector width): plain fp32 FMA over LDS tiles, any strides,
// every dtype of the C ABI.  Correct first, not fast; the semantics are those of the
// reference `matmul_kernel` (python/tutorials/03-matrix-multiplication.py:241-316): fp32
// accumulation, activation on the accumulator, one rounding to the output type.
#include "common.h"
#include "launch.h"
#include "formats.h"

namespace mi355 {

__device__ __forceinline__ float load_elem(const void* p, int64_t idx, int dtype) {
  switch (dtype) {
    case 0: return (float)((const _Float16*)p)[idx];
    case 1: return (float)((const __bf16*)p)[idx];
    case 2: return e4m3_to_f32(((const uint8_t*)p)[idx]);
    case 3: return e5m2_to_f32(((const uint8_t*)p)[idx]);
    default: return ((const float*)p)[idx];
  }
}

__device__ __forceinline__ void store_elem(void* p, int64_t idx, int dtype, float v) {
  switch (dtype) {
    case 0: ((_Float16*)p)[idx] = (_Float16)v; break;
    case 1: ((__bf16*)p)[idx] = (__bf16)v; break;
    case 2: ((uint8_t*)p)[idx] = f32_to_e4m3(v); break;
    case 3: ((uint8_t*)p)[idx] = f32_to_e5m2(v); break;
    default: ((float*)p)[idx] = v; break;
  }
}

constexpr int TS = 64;  // C tile edge
constexpr int TK = 16;  // K step

__global__ __launch_bounds__(256) void gemm_strided_kernel(GemmStridedArgs p) {
  __shared__ float sa[TK][TS + 1];
  __shared__ float sb[TK][TS + 1];
  const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
  const int m0 = blockIdx.y * TS, n0 = blockIdx.x * TS;
  float acc[4][4] = {};
  for (int k0 = 0; k0 < p.K; k0 += TK) {
    for (int i = threadIdx.x; i < TS * TK; i += 256) {
      int r = i / TK, kk = i % TK;
      int m = m0 + r, k = k0 + kk;
      sa[kk][r] = (m < p.M && k < p.K) ? load_elem(p.A, (int64_t)m * p.sam + (int64_t)k * p.sak, p.in_dtype) : 0.f;
      int kk2 = i / TS, c = i % TS;
      int n = n0 + c, k2 = k0 + kk2;
      sb[kk2][c] = (n < p.N && k2 < p.K) ? load_elem(p.B, (int64_t)k2 * p.sbk + (int64_t)n * p.sbn, p.in_dtype) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < TK; kk++) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; i++) a[i] = sa[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; j++) b[j] = sb[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
  float alpha = 1.f;
  if (p.a_scale) alpha *= *p.a_scale;
  if (p.b_scale) alpha *= *p.b_scale;
  for (int i = 0; i < 4; i++)
    for (int j = 0; j < 4; j++) {
      int m = m0 + ty * 4 + i, n = n0 + tx * 4 + j;
      if (m < p.M && n < p.N) {
        float x = acc[i][j] * alpha;
        if (p.aux) x += load_aux(p.aux, (int64_t)m * p.aux_sm + (int64_t)n * p.aux_sn, p.aux_dtype);
        if (p.activation == 1) x = x >= 0.f ? x : 0.01f * x;
        store_elem(p.C, (int64_t)m * p.scm + (int64_t)n * p.scn, p.out_dtype, x);
      }
    }
}

int gemm_strided_launch(const GemmStridedArgs& p, hipStream_t stream) {
  dim3 grid((p.N + TS - 1) / TS, (p.M + TS - 1) / TS);
  hipLaunchKernelGGL(gemm_strided_kernel, grid, dim3(256), 0, stream, p);
  return (int)hipGetLastError();
}

}  // namespace mi355

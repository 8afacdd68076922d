// GEMM for operands that the tiled MFMA kernels do not take - no unit stride, rows that are not whole 16-byte chunks
// (K or N not a multiple of the vector width), unaligned bases: any strides, any sizes, every type of the C ABI, the
// way the reference's kernel takes them with masked loads (python/tutorials/03-matrix-multiplication.py:281-298,
// :312-316).  Tiles of 64 x 64 on 32x32x16 MFMAs (four waves of 32 x 32), K steps of 32 elements; a thread fetches
// eight consecutive elements of one operand row per step - one 16-byte (fp8: 8-byte) load where those are contiguous,
// aligned and inside the matrix, eight masked element loads otherwise - a K step ahead of the MFMAs that use them,
// through registers into one of two LDS buffers.  fp8 operands are widened to fp16 on the way (exact for both fp8
// types), so every product and the fp32 accumulation are those of the fp8 kernels.  Semantics as everywhere: fp32
// accumulation, scales, addend and activation on the accumulator, one rounding to the output type.
#include "common.h"
#include "launch.h"
#include "formats.h"

namespace mi355 {

namespace {

constexpr int MBM = 64, MBN = 64, MBK = 32;
constexpr int PITCH = 40;   // elements per LDS row: 32 + 8, rows stay 16-byte aligned and eight rows fall on distinct banks

typedef uint16_t u16x8 __attribute__((ext_vector_type(8)));

// IN: 0 = fp16, 1 = bf16, 2 = e4m3, 3 = e5m2 (the C ABI's codes); the bits of the 16-bit element the MFMAs take
template <int IN>
__device__ __forceinline__ uint16_t widen(const void* base, int64_t idx) {
  if constexpr (IN <= 1) return ((const uint16_t*)base)[idx];
  else if constexpr (IN == 2) return __builtin_bit_cast(uint16_t, (_Float16)e4m3_to_f32(((const uint8_t*)base)[idx]));
  else return (uint16_t)(((const uint8_t*)base)[idx] << 8);   // e5m2 is the upper byte of the fp16 of the same value
}

// eight elements r, k .. k + 7 of an operand with element strides (s_row, s_k); zeros outside [0, rows) x [0, K)
template <int IN>
__device__ __forceinline__ u16x8 fetch8_along_k(const void* base, int64_t s_row, int64_t s_k, int r, int rows, int k, int K) {
  u16x8 v = {0, 0, 0, 0, 0, 0, 0, 0};
  if (r >= rows || k >= K) return v;
  constexpr int EB = IN <= 1 ? 2 : 1;
  const int64_t idx = (int64_t)r * s_row + (int64_t)k * s_k;
  if (s_k == 1 && k + 8 <= K && (((uintptr_t)base + idx * EB) % (8 * EB)) == 0) {
    if constexpr (IN <= 1) {
      return *(const u16x8*)((const uint16_t*)base + idx);
    } else {
      const uint64_t raw = *(const uint64_t*)((const uint8_t*)base + idx);
#pragma unroll
      for (int e = 0; e < 8; e++) {
        const uint8_t c = (uint8_t)(raw >> (8 * e));
        v[e] = IN == 2 ? __builtin_bit_cast(uint16_t, (_Float16)e4m3_to_f32(c)) : (uint16_t)(c << 8);
      }
      return v;
    }
  }
#pragma unroll
  for (int e = 0; e < 8; e++)
    if (k + e < K) v[e] = widen<IN>(base, idx + e * s_k);
  return v;
}

// eight elements k, c .. c + 7 of a [K, cols] operand whose columns are contiguous (s_c == 1); zeros outside
template <int IN>
__device__ __forceinline__ u16x8 fetch8_along_n(const void* base, int64_t s_k, int k, int K, int c, int cols) {
  u16x8 v = {0, 0, 0, 0, 0, 0, 0, 0};
  if (k >= K || c >= cols) return v;
  constexpr int EB = IN <= 1 ? 2 : 1;
  const int64_t idx = (int64_t)k * s_k + c;
  if (c + 8 <= cols && (((uintptr_t)base + idx * EB) % (8 * EB)) == 0) {
    if constexpr (IN <= 1) {
      return *(const u16x8*)((const uint16_t*)base + idx);
    } else {
      const uint64_t raw = *(const uint64_t*)((const uint8_t*)base + idx);
#pragma unroll
      for (int e = 0; e < 8; e++) {
        const uint8_t b = (uint8_t)(raw >> (8 * e));
        v[e] = IN == 2 ? __builtin_bit_cast(uint16_t, (_Float16)e4m3_to_f32(b)) : (uint16_t)(b << 8);
      }
      return v;
    }
  }
#pragma unroll
  for (int e = 0; e < 8; e++)
    if (c + e < cols) v[e] = widen<IN>(base, idx + e);
  return v;
}

__device__ __forceinline__ void store_out(void* p, int64_t idx, int dtype, float v) {
  switch (dtype) {
    case 0: ((_Float16*)p)[idx] = (_Float16)v; break;
    case 1: ((__bf16*)p)[idx] = (__bf16)v; break;
    case 2: ((uint8_t*)p)[idx] = f32_to_e4m3(v); break;
    case 3: ((uint8_t*)p)[idx] = f32_to_e5m2(v); break;
    default: ((float*)p)[idx] = v; break;
  }
}

template <int IN>
__global__ __launch_bounds__(256) void gemm_masked_kernel(GemmStridedArgs p) {
  using V8 = std::conditional_t<IN == 1, bf16x8, f16x8>;
  __shared__ __attribute__((aligned(16))) uint16_t sa[2][MBM * PITCH];
  __shared__ __attribute__((aligned(16))) uint16_t sb[2][MBN * PITCH];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1, l32 = lane & 31, g = lane >> 5;
  const int nbn = (p.N + MBN - 1) / MBN;   // (a one-dimensional grid: either count of tiles may exceed 65535)
  const int m0 = (int)(blockIdx.x / nbn) * MBM, n0 = (int)(blockIdx.x % nbn) * MBN;
  const bool b_rows_contiguous = p.sbn == 1 && p.sbk != 1;   // row-major B: fetch along n, store transposed

  // A and a B with any other layout: thread -> row tid / 4, elements 8 (tid % 4) .. + 7 of the K step;
  // row-major B: thread -> k row tid % 32, columns 8 (tid / 32) .. + 7
  const int fr = tid >> 2, fc = (tid & 3) * 8;
  const int bk = tid & 31, bc = (tid >> 5) * 8;
  auto fetch_a = [&](int k0) { return fetch8_along_k<IN>(p.A, p.sam, p.sak, m0 + fr, p.M, k0 + fc, p.K); };
  auto fetch_b = [&](int k0) {
    return b_rows_contiguous ? fetch8_along_n<IN>(p.B, p.sbk, k0 + bk, p.K, n0 + bc, p.N)
                             : fetch8_along_k<IN>(p.B, p.sbn, p.sbk, n0 + fr, p.N, k0 + fc, p.K);
  };
  auto stash = [&](int buf, u16x8 va, u16x8 vb) {
    *(u16x8*)&sa[buf][fr * PITCH + fc] = va;
    if (b_rows_contiguous) {
#pragma unroll
      for (int e = 0; e < 8; e++) sb[buf][(bc + e) * PITCH + bk] = vb[e];
    } else {
      *(u16x8*)&sb[buf][fr * PITCH + fc] = vb;
    }
  };

  f32x16 acc;
#pragma unroll
  for (int i = 0; i < 16; i++) acc[i] = 0.f;

  const int nsteps = (p.K + MBK - 1) / MBK;
  u16x8 va = fetch_a(0), vb = fetch_b(0);
  stash(0, va, vb);
  __syncthreads();
  for (int s = 0; s < nsteps; s++) {
    const int buf = s & 1;
    if (s + 1 < nsteps) { va = fetch_a((s + 1) * MBK); vb = fetch_b((s + 1) * MBK); }
#pragma unroll
    for (int kk = 0; kk < MBK / 16; kk++) {
      const V8 fa = __builtin_bit_cast(V8, *(const u16x8*)&sa[buf][(wm * 32 + l32) * PITCH + kk * 16 + g * 8]);
      const V8 fb = __builtin_bit_cast(V8, *(const u16x8*)&sb[buf][(wn * 32 + l32) * PITCH + kk * 16 + g * 8]);
      acc = mfma32(fa, fb, acc);   // register 4 rg + e of lane (l32, g): row 8 rg + 4 g + e, column l32
    }
    // (the other buffer was last read in the step before, which every wave left through the barrier below)
    if (s + 1 < nsteps) stash(buf ^ 1, va, vb);
    __syncthreads();
  }

  float alpha = 1.f;
  if (p.a_scale) alpha *= *p.a_scale;
  if (p.b_scale) alpha *= *p.b_scale;
  const int n = n0 + wn * 32 + l32;
  if (n >= p.N) return;
#pragma unroll
  for (int i = 0; i < 16; i++) {
    const int m = m0 + wm * 32 + (i >> 2) * 8 + g * 4 + (i & 3);
    if (m >= p.M) continue;
    float x = acc[i] * alpha;
    if (p.aux) x += load_aux(p.aux, (int64_t)m * p.aux_sm + (int64_t)n * p.aux_sn, p.aux_dtype);
    if (p.activation == 1) x = x >= 0.f ? x : 0.01f * x;
    store_out(p.C, (int64_t)m * p.scm + (int64_t)n * p.scn, p.out_dtype, x);
  }
}

}  // namespace

int gemm_masked_launch(const GemmStridedArgs& p, hipStream_t stream) {
  const int64_t tiles = (int64_t)((p.N + MBN - 1) / MBN) * ((p.M + MBM - 1) / MBM);
  if (tiles <= 0 || tiles > 0x7fffffffll) return -1;   // (MI355_EINVAL)
  dim3 grid((unsigned)tiles);
  switch (p.in_dtype) {
    case 0: hipLaunchKernelGGL(gemm_masked_kernel<0>, grid, dim3(256), 0, stream, p); break;
    case 1: hipLaunchKernelGGL(gemm_masked_kernel<1>, grid, dim3(256), 0, stream, p); break;
    case 2: hipLaunchKernelGGL(gemm_masked_kernel<2>, grid, dim3(256), 0, stream, p); break;
    default: hipLaunchKernelGGL(gemm_masked_kernel<3>, grid, dim3(256), 0, stream, p); break;
  }
  return (int)hipGetLastError();
}

}  // namespace mi355

// GEMM for operands that the tiled MFMA kernels do not take - no unit stride, rows that are not whole 16-byte chunks
// (K or N not a multiple of the vector width), unaligned bases: any strides, any sizes, every type of the C ABI, the
// way the reference's kernel takes them with masked loads (python/tutorials/03-matrix-multiplication.py:281-298,
// :312-316).  Tiles of 64 x 64 on 32x32x16 MFMAs (four waves of 32 x 32), K steps of 64 elements; a thread fetches
// two runs of eight consecutive elements of each operand per step - one load each where they are contiguous and
// inside the matrix, whatever their alignment; masked element loads otherwise - two K steps ahead of their MFMAs,
// through registers into one of two LDS buffers.  fp8 operands are widened to fp16 on the way (exact for both fp8
// types), so every product and the fp32 accumulation are those of the fp8 kernels.  Semantics as everywhere: fp32
// accumulation, scales, addend and activation on the accumulator, one rounding to the output type.
#include "common.h"
#include "launch.h"
#include "formats.h"

namespace mi355 {

namespace {

constexpr int MBM = 64, MBN = 64, MBK = 64;
constexpr int PITCH = 72;   // elements per LDS row: 64 + 8, rows stay 16-byte aligned and eight rows fall on distinct banks

typedef uint16_t u16x8 __attribute__((ext_vector_type(8)));

// IN: 0 = fp16, 1 = bf16, 2 = e4m3, 3 = e5m2 (the C ABI's codes).  Eight operand elements as they come from memory
// (16-bit types: the eight elements; fp8: eight codes in a 64-bit word) and as the MFMAs take them (fp8 widened to
// fp16: e5m2 is the upper byte of the fp16 of the same value, e4m3 goes through fp32).
template <int IN> struct Raw8 { using type = u16x8; };
template <> struct Raw8<2> { using type = uint64_t; };
template <> struct Raw8<3> { using type = uint64_t; };
template <int IN>
__device__ __forceinline__ u16x8 widen8(typename Raw8<IN>::type raw) {
  if constexpr (IN <= 1) return raw;
  else {
    u16x8 v;
#pragma unroll
    for (int e = 0; e < 8; e++) {
      const uint8_t c = (uint8_t)(raw >> (8 * e));
      v[e] = IN == 2 ? __builtin_bit_cast(uint16_t, (_Float16)e4m3_to_f32(c)) : (uint16_t)(c << 8);
    }
    return v;
  }
}
template <int IN>
__device__ __forceinline__ void put(typename Raw8<IN>::type& raw, int e, const void* base, int64_t idx) {
  if constexpr (IN <= 1) raw[e] = ((const uint16_t*)base)[idx];
  else raw |= (uint64_t)((const uint8_t*)base)[idx] << (8 * e);
}

// Elements idx, idx + step, ... of an operand, the first `valid` (0 .. 8) of eight, zeros behind them.  A full run of
// contiguous elements is ONE load whatever its alignment (a copy of 16 / 8 bytes from an address of element
// alignment: the compiler emits the load forms that are legal at that alignment) and nothing in this function looks
// at what it returns - a caller can have several of them in flight; partial runs (the ends of K and of rows) and
// strided elements are fetched one by one.
template <int IN>
__device__ __forceinline__ typename Raw8<IN>::type fetch8(const void* base, int64_t idx, int64_t step, int valid) {
  typename Raw8<IN>::type raw{};
  constexpr int EB = IN <= 1 ? 2 : 1;
  if (step == 1 && valid == 8) {
    __builtin_memcpy(&raw, (const char*)base + idx * EB, 8 * EB);
  } else if (valid > 0) {
#pragma unroll
    for (int e = 0; e < 8; e++)
      if (e < valid) put<IN>(raw, e, base, idx + e * step);
  }
  return raw;
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

  // A and a B with any other layout: thread -> row tid / 4, elements 8 (tid % 4) .. + 7 and 32 further of the K step;
  // row-major B: thread -> k row tid % 64, columns 8 (tid / 64) .. + 7 and 32 further
  const int fr = tid >> 2, fc = (tid & 3) * 8;
  const int bk = tid & 63, bc = (tid >> 6) * 8;
  using Raw = typename Raw8<IN>::type;
  struct Regs { Raw a[2], b[2]; };
  auto left = [](int have, int at) { return at >= have ? 0 : have - at < 8 ? have - at : 8; };   // of eight from `at` on
  auto fetch = [&](int k0) {
    Regs x;
#pragma unroll
    for (int h = 0; h < 2; h++) {
      const int k = k0 + fc + 32 * h;
      x.a[h] = fetch8<IN>(p.A, (int64_t)(m0 + fr) * p.sam + (int64_t)k * p.sak, p.sak, m0 + fr < p.M ? left(p.K, k) : 0);
      if (b_rows_contiguous) {
        const int n = n0 + bc + 32 * h;
        x.b[h] = fetch8<IN>(p.B, (int64_t)(k0 + bk) * p.sbk + n, 1, k0 + bk < p.K ? left(p.N, n) : 0);
      } else {
        x.b[h] = fetch8<IN>(p.B, (int64_t)(n0 + fr) * p.sbn + (int64_t)k * p.sbk, p.sbk, n0 + fr < p.N ? left(p.K, k) : 0);
      }
    }
    return x;
  };
  auto stash = [&](int buf, const Regs& x) {
#pragma unroll
    for (int h = 0; h < 2; h++) {
      *(u16x8*)&sa[buf][fr * PITCH + fc + 32 * h] = widen8<IN>(x.a[h]);
      const u16x8 vb = widen8<IN>(x.b[h]);
      if (b_rows_contiguous) {
#pragma unroll
        for (int e = 0; e < 8; e++) sb[buf][(bc + 32 * h + e) * PITCH + bk] = vb[e];
      } else {
        *(u16x8*)&sb[buf][fr * PITCH + fc + 32 * h] = vb;
      }
    }
  };

  f32x16 acc;
#pragma unroll
  for (int i = 0; i < 16; i++) acc[i] = 0.f;

  const int nsteps = (p.K + MBK - 1) / MBK;
  // two K steps of operands are on their way at any time: step s + 2 is requested at the top of step s and goes into
  // LDS at the end of step s + 1 (few workgroups with long K - a single row or column of C - are bound by how many
  // bytes they have in flight).  The two steps in front of the first MFMAs run through the same loop body, so the
  // fetch and the LDS store exist once in the code: under the reference's timing protocol, which flushes the caches
  // before every call, a small product pays for every instruction line it has to fetch.
  Regs xn{}, xf{};
  for (int s = -2; s < nsteps; s++) {
    const int buf = s & 1;
    if (s + 2 < nsteps) xf = fetch((s + 2) * MBK);
    if (s >= 0) {
#pragma unroll
      for (int kk = 0; kk < MBK / 16; kk++) {
        const V8 fa = __builtin_bit_cast(V8, *(const u16x8*)&sa[buf][(wm * 32 + l32) * PITCH + kk * 16 + g * 8]);
        const V8 fb = __builtin_bit_cast(V8, *(const u16x8*)&sb[buf][(wn * 32 + l32) * PITCH + kk * 16 + g * 8]);
        acc = mfma32(fa, fb, acc);   // register 4 rg + e of lane (l32, g): row 8 rg + 4 g + e, column l32
      }
    }
    // (xn holds step s + 1; its buffer was last read in step s - 1, which every wave left through a barrier)
    if (s + 1 >= 0 && s + 1 < nsteps) stash(buf ^ 1, xn);
    __syncthreads();
    xn = xf;
  }

  float alpha = 1.f;
  if (p.a_scale) alpha *= *p.a_scale;
  if (p.b_scale) alpha *= *p.b_scale;
  // The epilogue as a loop that is NOT unrolled, over accumulator values parked in LDS (a register array cannot be
  // indexed by a loop counter): scales, addend, activation and the store with its run-time choice of output type
  // exist once instead of sixteen times - code that a small product would fetch from memory for every call.
  float* const park = (float*)&sa[0][0] + tid;          // [16][256] floats: 16 KiB of the 18 KiB that held A
#pragma unroll
  for (int i = 0; i < 16; i++) park[i * 256] = acc[i];  // (every wave left the K loop through its last barrier)
  const int n = n0 + wn * 32 + l32;
  if (n >= p.N) return;
#pragma unroll 1
  for (int i = 0; i < 16; i++) {
    const int m = m0 + wm * 32 + (i >> 2) * 8 + g * 4 + (i & 3);
    if (m >= p.M) continue;
    float x = park[i * 256] * alpha;
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

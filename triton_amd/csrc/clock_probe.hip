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

// ---- MFMA burn: what the matrix pipes of this board sustain with nothing else in the way.  Every SIMD of every
// CU runs `waves` waves that issue one MFMA shape back to back (eight independent accumulator chains, operands in
// registers, no memory traffic); the operands are either pseudo-random bit patterns per lane - finite values of
// every magnitude, the switching activity of real data - or one constant.  Timed by the caller with events and
// sampled for watts and clock, this is the ceiling that a GEMM of that MFMA shape can approach under the board's
// power limit: the denominator for "fraction of what the board sustains" next to the nominal peak.
namespace mi355 {
namespace {

typedef __attribute__((ext_vector_type(8))) int burn_i32x8;

__device__ inline unsigned burn_rnd(unsigned x) { x ^= x << 13; x ^= x >> 17; x ^= x << 5; return x; }

// two bf16 bit patterns: random sign and mantissa, exponent 0x78 .. 0x7f (magnitudes 2^-7 .. 2, where N(0, 1) data lives)
__device__ inline unsigned burn_bf16_pair(unsigned& s) {
  s = burn_rnd(s);
  const unsigned lo = (s & 0x807f) | ((((s >> 7) & 7) + 0x78) << 7);
  s = burn_rnd(s);
  const unsigned hi = (s & 0x807f) | ((((s >> 7) & 7) + 0x78) << 7);
  return lo | (hi << 16);
}

// four e4m3fn codes, uniform over the finite ones (0x7f / 0xff, the NaNs, lose their lowest bit)
__device__ inline unsigned burn_e4m3_quad(unsigned& s) {
  s = burn_rnd(s);
  const unsigned m = s & 0x7f7f7f7fu;
  const unsigned nan = m & (m >> 1) & (m >> 2) & (m >> 3) & (m >> 4) & (m >> 5) & (m >> 6) & 0x01010101u;
  return s & ~nan;
}

template <int SHAPE>
__device__ __forceinline__ void burn_mfma32(f32x16& c, const burn_i32x8& a, const burn_i32x8& b, const i32x4& a4, const i32x4& b4, int sa, int sb) {
#if MI355_DEVICE_PASS
  if constexpr (SHAPE == 6)
    asm volatile("v_mfma_scale_f32_32x32x64_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel_hi:[0,0,0] cbsz:4 blgp:4" : "+a"(c) : "v"(a4), "v"(b4), "v"(sa), "v"(sb));
  else if constexpr (SHAPE == 0) asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a4), "v"(b4));
  else if constexpr (SHAPE == 2) asm volatile("v_mfma_f32_32x32x64_f8f6f4 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
  else asm volatile("v_mfma_f32_32x32x64_f8f6f4 %0, %1, %2, %0 cbsz:4 blgp:4" : "+a"(c) : "v"(a4), "v"(b4));
#endif
}
template <int SHAPE>
__device__ __forceinline__ void burn_mfma16(f32x4& c, const burn_i32x8& a, const burn_i32x8& b, const i32x4& a4, const i32x4& b4, int sa, int sb) {
#if MI355_DEVICE_PASS
  if constexpr (SHAPE == 7)
    asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel_hi:[0,0,0] cbsz:4 blgp:4" : "+a"(c) : "v"(a4), "v"(b4), "v"(sa), "v"(sb));
  else if constexpr (SHAPE == 1) asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a4), "v"(b4));
  else if constexpr (SHAPE == 3) asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
  else asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, %0 cbsz:4 blgp:4" : "+a"(c) : "v"(a4), "v"(b4));
#endif
}
// two idle slots behind the (vector) write of an accumulator, tied to it: an assembly MFMA must not read a register
// within two slots of a vector write, and the compiler, which keeps that distance for MFMAs it knows, cannot here
template <typename V>
__device__ __forceinline__ void burn_settle(V& c) {
#if MI355_DEVICE_PASS
  asm volatile("s_nop 1" : "+a"(c));
#endif
}
__device__ __forceinline__ void burn_settle_operands(burn_i32x8& a0, burn_i32x8& a1, burn_i32x8& b0, burn_i32x8& b1,
                                                     i32x4& c0, i32x4& c1, i32x4& d0, i32x4& d1, int& sa, int& sb) {
#if MI355_DEVICE_PASS
  asm volatile("s_nop 1" : "+v"(a0), "+v"(a1), "+v"(b0), "+v"(b1), "+v"(c0), "+v"(c1), "+v"(d0), "+v"(d1), "+v"(sa), "+v"(sb));
#endif
}
template <typename V>
__device__ __forceinline__ void burn_pin(V& c) {
#if MI355_DEVICE_PASS
  asm volatile("" : "+a"(c));
#endif
}

template <int SHAPE>
__global__ __launch_bounds__(256) void mfma_burn_kernel(float* sink, int iters, int random_operands) {
#if MI355_DEVICE_PASS
  unsigned s = threadIdx.x * 2654435761u + blockIdx.x * 97u + 1u;
  burn_i32x8 a[2], b[2];
#pragma unroll
  for (int i = 0; i < 2; i++)
#pragma unroll
    for (int e = 0; e < 8; e++) {
      if (SHAPE < 2) {                       // 16-bit operands: four registers used
        a[i][e] = random_operands ? (int)burn_bf16_pair(s) : 0x3f803f80;
        b[i][e] = random_operands ? (int)burn_bf16_pair(s) : 0x3f803f80;
      } else if (SHAPE < 4) {                // e4m3 bytes: every finite code (0x7f / 0xff, the NaNs, mapped away)
        a[i][e] = random_operands ? (int)burn_e4m3_quad(s) : 0x38383838;
        b[i][e] = random_operands ? (int)burn_e4m3_quad(s) : 0x38383838;
      } else {                               // e2m1 nibbles: every code is finite
        s = burn_rnd(s); a[i][e] = random_operands ? (int)s : 0x22222222;
        s = burn_rnd(s); b[i][e] = random_operands ? (int)s : 0x22222222;
      }
    }
  // The MFMAs are issued as assembly with the accumulators pinned to accumulation registers, as the GEMM kernels
  // issue theirs (left to the register allocator, the chains of four-register tiles were rotated through
  // architectural registers in every round, at half the rate).  16-bit and fp4 operands are four registers, fp8 eight.
  // block scales of the scaled fp4 legs (e8m0 in byte 0): 2^-4 .. 2^4, or 1
  s = burn_rnd(s);
  int sa = random_operands ? 123 + (int)(s % 9u) : 127, sb = random_operands ? 123 + (int)((s >> 8) % 9u) : 127;
  float total = 0.f;
  i32x4 a4[2] = {__builtin_shufflevector(a[0], a[0], 0, 1, 2, 3), __builtin_shufflevector(a[1], a[1], 0, 1, 2, 3)};
  i32x4 b4[2] = {__builtin_shufflevector(b[0], b[0], 0, 1, 2, 3), __builtin_shufflevector(b[1], b[1], 0, 1, 2, 3)};
  if constexpr (SHAPE == 0 || SHAPE == 2 || SHAPE == 4 || SHAPE == 6) {         // 32 x 32 tiles: four chains of 16 registers
    f32x16 acc[4];
#pragma unroll
    for (int c = 0; c < 4; c++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[c][r] = 0.f;
#pragma unroll
    for (int c = 0; c < 4; c++) burn_settle(acc[c]);
    burn_settle_operands(a[0], a[1], b[0], b[1], a4[0], a4[1], b4[0], b4[1], sa, sb);
    for (int i = 0; i < iters; i++) {
#pragma unroll
      for (int u = 0; u < 8; u++) burn_mfma32<SHAPE>(acc[u & 3], a[u & 1], b[(u >> 1) & 1], a4[u & 1], b4[(u >> 1) & 1], sa, sb);
    }
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");          // the last MFMAs retire before their results are read
#pragma unroll
    for (int c = 0; c < 4; c++) {
      burn_pin(acc[c]);
#pragma unroll
      for (int r = 0; r < 16; r++) total += acc[c][r];
    }
  } else {                                                         // 16 x 16 tiles: eight chains of 4 registers
    f32x4 acc[8];
#pragma unroll
    for (int c = 0; c < 8; c++)
#pragma unroll
      for (int r = 0; r < 4; r++) acc[c][r] = 0.f;
#pragma unroll
    for (int c = 0; c < 8; c++) burn_settle(acc[c]);
    burn_settle_operands(a[0], a[1], b[0], b[1], a4[0], a4[1], b4[0], b4[1], sa, sb);
    for (int i = 0; i < iters; i++) {
#pragma unroll
      for (int u = 0; u < 16; u++) burn_mfma16<SHAPE>(acc[u & 7], a[u & 1], b[(u >> 1) & 1], a4[u & 1], b4[(u >> 1) & 1], sa, sb);
    }
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
#pragma unroll
    for (int c = 0; c < 8; c++) {
      burn_pin(acc[c]);
#pragma unroll
      for (int r = 0; r < 4; r++) total += acc[c][r];
    }
  }
  if (total == 12345.678f) sink[0] = total;   // (keeps the chains alive; practically never true)
#endif
}

}  // namespace

// flop of one launch: every shape's inner loop is 8 x 32768 (16-bit), x2 (fp8), x4 (fp4) flop per wave and iteration
int mfma_burn_launch(float* sink, int shape, int random_operands, int iters, int waves_per_simd, int cus, hipStream_t stream) {
  const dim3 grid(cus * waves_per_simd), block(256);
  switch (shape) {
    case 0: hipLaunchKernelGGL(mfma_burn_kernel<0>, grid, block, 0, stream, sink, iters, random_operands); break;
    case 1: hipLaunchKernelGGL(mfma_burn_kernel<1>, grid, block, 0, stream, sink, iters, random_operands); break;
    case 2: hipLaunchKernelGGL(mfma_burn_kernel<2>, grid, block, 0, stream, sink, iters, random_operands); break;
    case 3: hipLaunchKernelGGL(mfma_burn_kernel<3>, grid, block, 0, stream, sink, iters, random_operands); break;
    case 4: hipLaunchKernelGGL(mfma_burn_kernel<4>, grid, block, 0, stream, sink, iters, random_operands); break;
    case 5: hipLaunchKernelGGL(mfma_burn_kernel<5>, grid, block, 0, stream, sink, iters, random_operands); break;
    case 6: hipLaunchKernelGGL(mfma_burn_kernel<6>, grid, block, 0, stream, sink, iters, random_operands); break;
    case 7: hipLaunchKernelGGL(mfma_burn_kernel<7>, grid, block, 0, stream, sink, iters, random_operands); break;
    default: return -1;
  }
  return (int)hipGetLastError();
}

}  // namespace mi355

// Pieces shared by the four-wave GEMM kernels (gemm_wave128.hip: 16-bit and fp8; gemm_wave128_mx.hip: the
// block-scaled forms): the wait for the last MFMAs, the grid size, and the epilogue of 16x16 accumulator tiles.
#pragma once

// L2 touches ahead of the direct loads in the four-wave kernels (see gemm_wave128_tiles): on / off and the number of
// K steps they run ahead of the loads, as build-time switches for A/B measurements.
#ifndef MI355_W128_PREFETCH
#define MI355_W128_PREFETCH 1
#endif
#ifndef MI355_W128_PREFETCH_DISTANCE
#define MI355_W128_PREFETCH_DISTANCE 2
#endif
#include "gemm_core.h"

namespace mi355 {

// Epilogue for 16x16 tiles computed with the operands swapped (D[n][m]): lane l owns C row
// `mrow0 + 16 i + l%16` and, of tile (i, j), the four consecutive columns `ncol0 + 16 j + 4 (l/16) ..`.
// The MFMAs of these kernels are inline assembly, so the compiler neither knows that they are MFMAs nor waits
// for the last ones before it reads their results.  Waiting alone is not enough: nothing ties a plain
// `s_nop` statement to the accumulators, and the compiler has moved accumulator reads (spills and moves of the
// epilogue's register shuffle) in front of it, where they see registers that the last MFMAs have yet to write.
// So every accumulator passes through an (empty) assembly statement behind the wait: volatile statements keep
// their order, and a value read after its statement is read after the wait.
//
// The wait itself (mfma_retire) stands INSIDE the K loop, at the end of the body of a tile's last iteration:
// whatever the register allocator does with the accumulators on the edge that leaves the loop (its register
// shuffle for the epilogue, spills), it does behind the loop's last basic block, hence behind the wait.  A
// wait placed behind the loop can end up behind those moves (a block-scaled fp8 product once came out wrong
// that way, in one run of many).  A read of an MFMA result has to come (passes + 3) issue slots behind the
// MFMA - 7 for the 4-pass 16x16x32 16-bit and 16x16x128 fp4 forms, 11 for the 8-pass 16x16x128 fp8 form -;
// `s_nop 15` is 16 slots of 4 cycles, once per tile.
// The loop compares with a copy of the step count that went through an empty assembly statement: told that
// the test equals the loop's own exit test, the compiler sinks the wait out of the loop again.
__device__ __forceinline__ void mfma_retire() {
#if MI355_DEVICE_PASS
  asm volatile("s_nop 15" ::: "memory");
#endif
}
__device__ __forceinline__ void mfma_drain_row(f32x4 (&r)[8]) {
#if MI355_DEVICE_PASS
  asm volatile("" : "+a"(r[0]), "+a"(r[1]), "+a"(r[2]), "+a"(r[3]), "+a"(r[4]), "+a"(r[5]), "+a"(r[6]), "+a"(r[7]));
#endif
}
template <int MT>
__device__ __forceinline__ void mfma_drain(f32x4 (&acc)[MT][8]) {
#if MI355_DEVICE_PASS
  asm volatile("s_nop 15" ::: "memory");
#endif
#pragma unroll
  for (int i = 0; i < MT; i++) mfma_drain_row(acc[i]);
}

// Workgroups for `tiles` tiles on at most `cap` CUs.  More tiles than CUs need r = ceil(tiles / cap) rounds
// however they are dealt: ceil(tiles / r) programs walk r tiles each (the last ones r - 1) as one stream of K
// steps, without the restart that a fresh workgroup per tile pays, and the CUs left without a program leave
// their share of the board's power to the others.  Against one workgroup per tile wherever the tiles do not
// divide by the CU count, same call, bf16 / fp8 TFLOP/s: 6144^3 (576 tiles -> 192 programs) 1240 vs 1180 and
// 2380 vs 2200; 7168^3 (784 -> 196) 1270 vs 1200 and 2450 vs 2307; 4352 x 4352 x 4096 (289 -> 145) 973 vs 892
// and 1692 vs 1603; 5120^3 (400 -> 200) 1233 vs 1229 and 2323 vs 2248; 4096 x 11008 x 4096 (688 -> 230, ragged)
// 1315 vs 1307 and 2408 vs 2330.
static inline int wave128_grid(int tiles, int cap) {
  if (cap <= 0 || tiles <= cap) return tiles;
  const int rounds = (tiles + cap - 1) / cap;
  return (tiles + rounds - 1) / rounds;
}

// AuxT: element type of the addend of the fused epilogues (void = none).  With an addend the kernels are
// separate instantiations: its arguments cost the plain kernels scalar registers that they need for their
// load bases.  `aux_vec`: the four addend elements of a lane are consecutive and aligned (one load).
template <int MT, int NT, typename AuxT>
__device__ __forceinline__ void gemm_epilogue16_impl(f32x4 (&acc)[MT][NT], const GemmArgs& p, int mrow0, int ncol0, int l16, int kg) {
  constexpr bool AUX = !std::is_void<AuxT>::value;
  using AuxE = std::conditional_t<AUX, AuxT, float>;
  typedef AuxE Aux4 __attribute__((ext_vector_type(4)));
  float alpha = 1.f;
  if (p.a_scale) alpha *= *p.a_scale;
  if (p.b_scale) alpha *= *p.b_scale;
  const bool leaky = p.activation == 1;
  const bool aux_vec = AUX && p.aux_sn == 1 && p.aux_sm % 4 == 0 && (uintptr_t)p.aux % 16 == 0;
  static_for<MT>([&](auto I_) {
    constexpr int i = decltype(I_)::value;
    const int m = mrow0 + i * 16 + l16;
    static_for<NT>([&](auto J_) {
      constexpr int j = decltype(J_)::value;
      const int n = ncol0 + j * 16 + kg * 4;
      float v[4];
#pragma unroll
      for (int e = 0; e < 4; e++) v[e] = acc[i][j][e] * alpha;
      if constexpr (AUX) {
        const AuxE* ax = (const AuxE*)p.aux + (int64_t)m * p.aux_sm + (int64_t)n * p.aux_sn;
        if (aux_vec) {
          const Aux4 t = *(const Aux4*)ax;
#pragma unroll
          for (int e = 0; e < 4; e++) v[e] += (float)t[e];
        } else {
#pragma unroll
          for (int e = 0; e < 4; e++) v[e] += (float)ax[e * p.aux_sn];
        }
      }
      if (leaky) {
#pragma unroll
        for (int e = 0; e < 4; e++) v[e] = v[e] >= 0.f ? v[e] : 0.01f * v[e];
      }
      if (p.out_dtype == 2 || p.out_dtype == 3) {
        store4_fp8(p.C, (int64_t)m * p.ldc + (int64_t)n * p.scn, p.scn, p.out_dtype, v, p.c_vec_ok, 4);
      } else if (p.out_dtype == 4) {
        float* c = (float*)p.C + (int64_t)m * p.ldc + (int64_t)n * p.scn;
        if (p.c_vec_ok) *(f32x4*)c = f32x4{v[0], v[1], v[2], v[3]};
        else {
#pragma unroll
          for (int e = 0; e < 4; e++) c[e * p.scn] = v[e];
        }
      } else if (p.out_dtype == 1) {
        __bf16* c = (__bf16*)p.C + (int64_t)m * p.ldc + (int64_t)n * p.scn;
        if (p.c_vec_ok) *(bf16x4*)c = bf16x4{(__bf16)v[0], (__bf16)v[1], (__bf16)v[2], (__bf16)v[3]};
        else {
#pragma unroll
          for (int e = 0; e < 4; e++) c[e * p.scn] = (__bf16)v[e];
        }
      } else {
        _Float16* c = (_Float16*)p.C + (int64_t)m * p.ldc + (int64_t)n * p.scn;
        if (p.c_vec_ok) *(f16x4*)c = f16x4{(_Float16)v[0], (_Float16)v[1], (_Float16)v[2], (_Float16)v[3]};
        else {
#pragma unroll
          for (int e = 0; e < 4; e++) c[e * p.scn] = (_Float16)v[e];
        }
      }
    });
  });
}

template <int MT, int NT, bool AUX = false>
__device__ __forceinline__ void gemm_epilogue16(f32x4 (&acc)[MT][NT], const GemmArgs& p, int mrow0, int ncol0, int l16, int kg) {
  if constexpr (!AUX) gemm_epilogue16_impl<MT, NT, void>(acc, p, mrow0, ncol0, l16, kg);
  else if (p.aux_dtype == 4) gemm_epilogue16_impl<MT, NT, float>(acc, p, mrow0, ncol0, l16, kg);
  else if (p.aux_dtype == 1) gemm_epilogue16_impl<MT, NT, __bf16>(acc, p, mrow0, ncol0, l16, kg);
  else gemm_epilogue16_impl<MT, NT, _Float16>(acc, p, mrow0, ncol0, l16, kg);
}

// The same for a plain C = A @ B in the operands' own 16-bit type with unit column stride (the grouped GEMM).
template <int MT, int NT, typename OutT>
__device__ __forceinline__ void gemm_epilogue16_plain(f32x4 (&acc)[MT][NT], const GemmArgs& p, int mrow0, int ncol0, int l16, int kg) {
  typedef OutT Out4 __attribute__((ext_vector_type(4)));
  static_for<MT>([&](auto I_) {
    constexpr int i = decltype(I_)::value;
    OutT* row = (OutT*)p.C + (int64_t)(mrow0 + i * 16 + l16) * p.ldc + ncol0 + kg * 4;
    static_for<NT>([&](auto J_) {
      constexpr int j = decltype(J_)::value;
      const f32x4 v = acc[i][j];
      if (p.c_vec_ok) *(Out4*)(row + j * 16) = Out4{(OutT)v[0], (OutT)v[1], (OutT)v[2], (OutT)v[3]};
      else {
#pragma unroll
        for (int e = 0; e < 4; e++) row[j * 16 + e] = (OutT)v[e];
      }
    });
  });
}

// The common case as an epilogue of its own: C in a 16-bit type with unit column stride and aligned rows, the
// product scaled by the per-tensor scales (1 without), no activation, no addend.  The general epilogue above decides
// output type, activation and store form at run time inside its 64 unrolled tiles, which makes it 70 KiB of code -
// more than the instruction cache holds, fetched anew at the end of every tile (and from memory when the kernel
// starts on cold caches): same call, 8192^3 bf16 1425 -> 1457 TFLOP/s back to back and 1352 -> 1397 with flushed
// caches, 4096^3 1201 -> 1301 and 1011 -> 1205.  Kernels take it as a separate instantiation, chosen on the host.
// A lane holds 4 consecutive columns of a 16-column tile (8 bytes of C), so stores straight from the registers are 64
// pieces of 8 bytes per instruction and the memory pipeline takes a request per piece: 16384 of them per 256 x 256
// tile.  Two neighbouring tiles are therefore exchanged between the lane pairs (kg, kg ^ 1) first
// (v_permlane16_swap: the odd 16-lane rows of its first register with the even rows of its second): the even lane
// then holds 8 consecutive columns of the first tile and the odd lane 8 of the second - 16 bytes per lane, half the
// requests and half the store instructions (rows need 16-byte alignment: lean_epilogue_type).
__device__ __forceinline__ void swap16(int& a, int& b) {
#if MI355_DEVICE_PASS
  asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(a), "+v"(b));
#endif
}
template <int MT, int NT, typename OutT>
__device__ __forceinline__ void gemm_epilogue16_lean(f32x4 (&acc)[MT][NT], const GemmArgs& p, int mrow0, int ncol0, int l16, int kg) {
  static_assert(NT % 2 == 0 && sizeof(OutT) == 2, "pairs of 16-column tiles of a 16-bit type");
  typedef OutT Out2 __attribute__((ext_vector_type(2)));
  float alpha = 1.f;
  if (p.a_scale) alpha *= *p.a_scale;
  if (p.b_scale) alpha *= *p.b_scale;
  // even kg: columns 4 kg .. 4 kg + 7 of the pair's first tile; odd kg: 4 (kg - 1) .. 4 (kg - 1) + 7 of its second
  const int col = ncol0 + 4 * (kg & 2) + 16 * (kg & 1);
  static_for<MT>([&](auto I_) {
    constexpr int i = decltype(I_)::value;
    OutT* row = (OutT*)p.C + (int64_t)(mrow0 + i * 16 + l16) * p.ldc + col;
    static_for<NT / 2>([&](auto J_) {
      constexpr int j = 2 * decltype(J_)::value;
      const f32x4 u = acc[i][j], v = acc[i][j + 1];
      int a0 = __builtin_bit_cast(int, Out2{(OutT)(u[0] * alpha), (OutT)(u[1] * alpha)});
      int a1 = __builtin_bit_cast(int, Out2{(OutT)(u[2] * alpha), (OutT)(u[3] * alpha)});
      int b0 = __builtin_bit_cast(int, Out2{(OutT)(v[0] * alpha), (OutT)(v[1] * alpha)});
      int b1 = __builtin_bit_cast(int, Out2{(OutT)(v[2] * alpha), (OutT)(v[3] * alpha)});
      swap16(a0, b0);
      swap16(a1, b1);
      *(i32x4*)(row + j * 16) = i32x4{a0, a1, b0, b1};
    });
  });
}
// 0 = the problem needs the general epilogue; else the C ABI code + 1 of the 16-bit output type the lean one writes
static inline int lean_epilogue_type(const GemmArgs& p) {
  if (!p.lean_ok || p.aux || p.activation != 0 || p.scn != 1 || !p.c_vec_ok || p.ldc % 8 != 0) return 0;
  return p.out_dtype == 0 ? 1 : p.out_dtype == 1 ? 2 : 0;
}

}  // namespace mi355

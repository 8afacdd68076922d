// Shared device-side helpers for the gfx950 kernels: vector types, MFMA wrappers,
// LDS swizzles, direct global->LDS tile copies and fp32 -> 16-bit conversions.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <utility>
#include <type_traits>

namespace mi355 {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(4))) _Float16 f16x4;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(8))) short s16x8;
typedef __attribute__((ext_vector_type(2))) int i32x2;
typedef __attribute__((ext_vector_type(4))) int i32x4;
typedef __attribute__((ext_vector_type(8))) int i32x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;

#define LDS_PTR(T) T __attribute__((address_space(3)))*

struct bf16_t { using vec8 = bf16x8; using vec4 = bf16x4; using scalar = __bf16; };
struct f16_t  { using vec8 = f16x8;  using vec4 = f16x4;  using scalar = _Float16; };

// D(32x32 fp32) += A(32x16) * B(16x32).  Lane l supplies A[l%32][8*(l/32) .. +8] and
// B[8*(l/32) .. +8][l%32]; accumulator register r of lane l is D[(r/4)*8 + 4*(l/32) + r%4][l%32].
__device__ __forceinline__ f32x16 mfma32(bf16x8 a, bf16x8 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ f32x16 mfma32(f16x8 a, f16x8 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
}

// fp32 -> 16-bit, round to nearest even (the compiler emits v_cvt_pk_bf16_f32 / v_cvt_f16_f32).
template <typename S> __device__ __forceinline__ S cvt16(float x) { return (S)x; }

// Builtins that need gfx950 target features are hidden from hipcc's host pass: a kernel
// template that reaches one there silently loses its host-side launch stub.
#if defined(__HIP_DEVICE_COMPILE__)
#define MI355_DEVICE_PASS 1
#else
#define MI355_DEVICE_PASS 0
#endif

// 16 bytes per lane straight from global memory into LDS: lane i of the wave writes
// lds_wave_base + 16 * i (the LDS address is wave-uniform, the global address per lane).
__device__ __forceinline__ void async_copy16(const void* gsrc, LDS_PTR(void) lds_wave_base) {
#if MI355_DEVICE_PASS
  __builtin_amdgcn_global_load_lds(gsrc, lds_wave_base, 16, 0, 0);
#endif
}

// The same copy with the global address split into a wave-uniform 64-bit base (scalar registers)
// and a 32-bit per-lane byte offset: the address add happens in the memory pipeline instead of
// costing a 64-bit vector add per load.  `lds_wave_base` must be wave-uniform.  The load is
// invisible to the compiler's wait-count bookkeeping: callers wait with wait_vmcnt<>.
// The statement writes M0 behind the compiler's back (M0 is a reserved register: a clobber is not honoured), and
// the compiler sets M0 itself for the LDS-direct loads it generates from the builtin (async_copy4 / async_copy16)
// and is free to move that write across this statement - the builtin's load then lands at this copy's address.
// A kernel therefore uses EITHER the builtin forms OR the inline-assembly forms (async_copy4_asm for 4 bytes),
// never both; tests/test_isa_hazards.py checks on the generated code that every LDS-direct load sees an M0
// written by its own side.
//
// SETTLE: a vector-memory instruction must not read a scalar register within 5 issue slots of a VALU
// instruction writing it - and that is how the compiler restores a SPILLED scalar register (v_readlane_b32),
// possibly right in front of this statement, whose contents it cannot see.  Inside the K loops the bases are
// produced by scalar arithmetic (checked on the generated code by tests/test_isa_hazards.py); the loads of a
// kernel's prologue, where restored spills do occur, are issued with SETTLE = true: five idle slots first.
template <bool SETTLE = false>
__device__ __forceinline__ void async_copy16_sbase(const void* sbase, unsigned lane_off, unsigned lds_wave_base) {
#if MI355_DEVICE_PASS
  // one idle issue slot between the M0 write and the LDS-DMA instruction that reads it
  if constexpr (SETTLE)
    asm volatile("s_nop 4\n\ts_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                 :: "v"(lane_off), "s"(sbase), "s"(lds_wave_base) : "memory");
  else
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                 :: "v"(lane_off), "s"(sbase), "s"(lds_wave_base) : "memory");
#endif
}

// The same with an instruction offset, which the hardware adds to BOTH addresses (global and LDS):
// several copies can then share one M0 value.  SETM0 = false reuses the M0 of the previous copy: nothing in
// between may write M0 (compiler-generated code does so only for indirect register indexing, message and GWS
// instructions and its own LDS-direct loads, none of which the kernels using this have).
template <int OFF, bool SETM0, bool SETTLE = false>
__device__ __forceinline__ void async_copy16_sbase_off(const void* sbase, unsigned lane_off, unsigned lds_wave_base) {
#if MI355_DEVICE_PASS
  // (SETTLE: see async_copy16_sbase; the idle slots stand inside the statement, behind any restore of its inputs)
  if constexpr (SETM0 && SETTLE)
    asm volatile("s_nop 4\n\ts_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 offset:%3"
                 :: "v"(lane_off), "s"(sbase), "s"(lds_wave_base), "i"(OFF) : "memory");
  else if constexpr (SETM0)
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 offset:%3"
                 :: "v"(lane_off), "s"(sbase), "s"(lds_wave_base), "i"(OFF) : "memory");
  else if constexpr (SETTLE)
    asm volatile("s_nop 4\n\tglobal_load_lds_dwordx4 %0, %1 offset:%2" :: "v"(lane_off), "s"(sbase), "i"(OFF) : "memory");
  else
    asm volatile("global_load_lds_dwordx4 %0, %1 offset:%2" :: "v"(lane_off), "s"(sbase), "i"(OFF) : "memory");
#endif
}

// A touch of one dword per lane, lanes 0 .. NLANES-1 only, at (wave-uniform 64-bit base + 32-bit lane offset),
// landing in 256 bytes of LDS that nobody reads: brings those lanes' cache lines into the L2 ahead of the loads that
// want them.  Counts in vmcnt like any load; sets M0 like the copies above (SETM0) or uses the value a preceding
// touch has set.  Only for code in which all 64 lanes are active: the execution mask is narrowed for the one
// instruction (every lane is a request to the cache, wanted or not) and set back to all lanes.
template <bool SETM0, int NLANES>
__device__ __forceinline__ void touch_line_sbase(const void* sbase, unsigned lane_off, unsigned lds_junk) {
#if MI355_DEVICE_PASS
  static_assert(NLANES >= 1 && NLANES <= 32, "lane mask as a 32-bit literal");
  constexpr unsigned MASK = NLANES == 32 ? 0xffffffffu : ((1u << NLANES) - 1u);
  if constexpr (SETM0)
    asm volatile("s_mov_b32 m0, %2\n\ts_mov_b64 exec, %3\n\tglobal_load_lds_dword %0, %1\n\ts_mov_b64 exec, -1"
                 :: "v"(lane_off), "s"(sbase), "s"(lds_junk), "i"(MASK) : "memory");
  else
    asm volatile("s_mov_b64 exec, %2\n\tglobal_load_lds_dword %0, %1\n\ts_mov_b64 exec, -1"
                 :: "v"(lane_off), "s"(sbase), "i"(MASK) : "memory");
#endif
}

// 16 bytes per lane from (wave-uniform 64-bit base + 32-bit lane offset + immediate) into
// registers, issued as inline assembly so that the compiler neither counts it nor waits for it:
// for loops that keep many loads in flight and wait with wait_vmcnt<> by hand.  The result may be
// used only after such a wait followed by lds_use() on the register.
template <int OFF, typename V>
__device__ __forceinline__ void load16_sbase(V& dst, const void* sbase, unsigned lane_off) {
  static_assert(sizeof(V) == 16 && OFF >= 0 && OFF < 4096, "one 16-byte register group, 12-bit offset");
#if MI355_DEVICE_PASS
  asm volatile("global_load_dwordx4 %0, %1, %2 offset:%3" : "=v"(dst) : "v"(lane_off), "s"(sbase), "i"(OFF));
#endif
}

// 4 bytes per lane, same addressing: lane i writes lds_wave_base + 4 * i.
__device__ __forceinline__ void async_copy4(const void* gsrc, LDS_PTR(void) lds_wave_base) {
#if MI355_DEVICE_PASS
  __builtin_amdgcn_global_load_lds(gsrc, lds_wave_base, 4, 0, 0);
#endif
}

// The same as one inline-assembly statement, for kernels whose other LDS-direct copies are inline assembly (see
// async_copy16_sbase: the compiler must not own M0 anywhere in such a kernel).  Not counted by the compiler: wait
// with wait_vmcnt<>.
__device__ __forceinline__ void async_copy4_asm(const void* gsrc, unsigned lds_wave_base) {
#if MI355_DEVICE_PASS
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off" :: "v"(gsrc), "s"(lds_wave_base) : "memory");
#endif
}

// 2^x by the hardware transcendental unit (denormal results flush to zero, as the reference
// allows on AMD: python/tutorials/06-fused-attention.py:452-454 `allow_flush_denorm`).
__device__ __forceinline__ float fast_exp2(float x) {
#if MI355_DEVICE_PASS
  return __builtin_amdgcn_exp2f(x);
#else
  return x;
#endif
}

// Exchange between the two lanes (l, l+32) that share a row of a 32x32 MFMA accumulator.
// v_permlane32_swap exchanges the upper half of its first register with the lower half of its
// second; fed with two copies of x it leaves (own, partner) in lanes < 32 and (partner, own)
// in lanes >= 32.  Issued as inline assembly (with the two wait states the instruction needs
// after a VALU write of its operands): the compiler builtin folds the two results into one.
__device__ __forceinline__ void swap32(float x, float& r0, float& r1) {
  float a = x, b = x;
#if MI355_DEVICE_PASS
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
#endif
  r0 = a;
  r1 = b;
}
// The same exchange on two registers of the caller: the upper half (lanes 32 .. 63) of `a` with the lower half of `b`.
__device__ __forceinline__ void swap32_regs(int& a, int& b) {
#if MI355_DEVICE_PASS
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
#endif
}
__device__ __forceinline__ float pair_max(float x) { float a, b; swap32(x, a, b); return fmaxf(a, b); }
__device__ __forceinline__ float pair_sum(float x) { float a, b; swap32(x, a, b); return a + b; }

// Compile-time counted loop: f(std::integral_constant<int, 0>) ... f(<N-1>), so that loop indices
// can be used as template arguments / instruction immediates.
template <typename F, int... Is>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, Is...>) {
  (f(std::integral_constant<int, Is>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(f, std::make_integer_sequence<int, N>{});
}

// LDS fragment reads issued as inline assembly.  The compiler cannot tell that a transpose
// read of one LDS stage does not alias an in-flight direct global->LDS load into the other
// stage and would wait for all outstanding loads first; reads it does not see are not
// delayed.  The price is that their completion has to be awaited by hand: lds_wait<N>()
// blocks until at most N LDS operations are outstanding, and lds_use(x) pins a register
// written by such a read so that no consumer is scheduled before the wait.
// (Hidden from the host pass like the builtins above.)
template <int OFF>
__device__ __forceinline__ i32x4 lds_read_b128(unsigned addr) {
  i32x4 v = {};
#if MI355_DEVICE_PASS
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "i"(OFF));
#endif
  return v;
}
template <int OFF>
__device__ __forceinline__ int lds_read_b32(unsigned addr) {
  int v = 0;
#if MI355_DEVICE_PASS
  asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "i"(OFF));
#endif
  return v;
}
template <int OFF>
__device__ __forceinline__ int lds_read_u16(unsigned addr) {   // two bytes, zero-extended
  int v = 0;
#if MI355_DEVICE_PASS
  asm volatile("ds_read_u16 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "i"(OFF));
#endif
  return v;
}
template <int OFF>
__device__ __forceinline__ int lds_read_u8(unsigned addr) {   // one byte, zero-extended
  int v = 0;
#if MI355_DEVICE_PASS
  asm volatile("ds_read_u8 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "i"(OFF));
#endif
  return v;
}
template <int OFF>
__device__ __forceinline__ i32x2 lds_read_tr16_b64(unsigned addr) {
  i32x2 v = {};
#if MI355_DEVICE_PASS
  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "i"(OFF));
#endif
  return v;
}
template <int OFF>
__device__ __forceinline__ i32x2 lds_read_tr8_b64(unsigned addr) {
  i32x2 v = {};
#if MI355_DEVICE_PASS
  asm volatile("ds_read_b64_tr_b8 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "i"(OFF));
#endif
  return v;
}
template <int N>
__device__ __forceinline__ void lds_wait() {
#if MI355_DEVICE_PASS
  // the counter has 4 bits; asking for "at most 15" where more are in flight only waits longer
  asm volatile("s_waitcnt lgkmcnt(%0)" ::"i"(N > 15 ? 15 : N));
#endif
}
template <typename V>
__device__ __forceinline__ void lds_use(V& v) {
#if MI355_DEVICE_PASS
  asm volatile("" : "+v"(v));
#endif
}
__device__ __forceinline__ unsigned lds_addr(LDS_PTR(const void) p) { return (unsigned)(uintptr_t)p; }

__device__ __forceinline__ void wait_all() { __builtin_amdgcn_s_waitcnt(0); }

// Wait until at most N vector-memory operations (loads, direct global->LDS copies) of this wave
// are outstanding; they complete in issue order.  vmcnt is split over bits 3:0 and 15:14 of the
// immediate, the other counters are left at "no wait".
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  static_assert(N >= 0 && N < 64, "vmcnt has 6 bits");
  __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | 0x0F70);
}

// Workgroup barrier WITHOUT the full memory wait the compiler puts in front of its own barrier:
// the K loops keep younger direct loads in flight across it.  The caller waits (wait_vmcnt /
// lds_wait) for exactly what the other waves are about to read.
__device__ __forceinline__ void block_barrier() {
#if MI355_DEVICE_PASS
  asm volatile("s_barrier" ::: "memory");
#endif
}

// Four fp32 values -> four fp8 codes in one dword (value 0 in the low byte), round to nearest even, by the
// hardware conversion (OCP e4m3fn / e5m2 on gfx950).  Values beyond the largest finite code come out as
// NaN (e4m3fn) / infinity (e5m2): callers that need saturation clamp first (pack4_fp8_sat).
template <int FMT>  // 0 = e4m3fn, 1 = e5m2
__device__ __forceinline__ int pack4_fp8(float a, float b, float c, float d) {
#if MI355_DEVICE_PASS
  int w = 0;
  if constexpr (FMT == 1) {
    w = __builtin_amdgcn_cvt_pk_bf8_f32(a, b, w, false);
    w = __builtin_amdgcn_cvt_pk_bf8_f32(c, d, w, true);
  } else {
    w = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, w, false);
    w = __builtin_amdgcn_cvt_pk_fp8_f32(c, d, w, true);
  }
  return w;
#else
  return 0;
#endif
}

// The same with finite overflow saturating to the largest finite code (448 / 57344, the downcast maxima of
// python/test/unit/language/test_conversions.py:307-329); NaN stays NaN.
template <int FMT>
__device__ __forceinline__ int pack4_fp8_sat(float a, float b, float c, float d) {
  constexpr float MAXV = FMT == 1 ? 57344.f : 448.f;
  auto sat = [](float x) { return x != x ? x : fminf(fmaxf(x, -MAXV), MAXV); };
  return pack4_fp8<FMT>(sat(a), sat(b), sat(c), sat(d));
}

// Store of four consecutive C elements as fp8 (out_dtype 2 = e4m3fn, 3 = e5m2): one dword when `vec`
// (unit column stride, 4-byte aligned), else `count` single bytes `scn` apart.
__device__ __forceinline__ void store4_fp8(char* C, int64_t off, int64_t scn, int out_dtype, const float (&v)[4], bool vec, int count) {
  const int w = out_dtype == 3 ? pack4_fp8_sat<1>(v[0], v[1], v[2], v[3]) : pack4_fp8_sat<0>(v[0], v[1], v[2], v[3]);
  if (vec && count == 4) {
    *(int*)(C + off) = w;
  } else {
#pragma unroll
    for (int e = 0; e < 4; e++)
      if (e < count) C[off + e * scn] = (char)(w >> (8 * e));
  }
}

// One element of the epilogue addend (dtype codes of the C ABI: 0 fp16, 1 bf16, 4 fp32).
__device__ __forceinline__ float load_aux(const void* aux, int64_t off, int dtype) {
  if (dtype == 4) return ((const float*)aux)[off];
  if (dtype == 1) return (float)((const __bf16*)aux)[off];
  return (float)((const _Float16*)aux)[off];
}

// Map a hardware workgroup id to a logical one so that ids that are consecutive in the
// logical order run on the same XCD (hardware deals workgroups round-robin over 8 XCDs,
// each with its own L2).
__device__ __forceinline__ int xcd_remap(int pid, int total) {
  constexpr int X = 8;
  int per = (total + X - 1) / X;
  int tall = total % X;
  int xcd = pid % X, local = pid / X;
  if (tall == 0 || xcd < tall) return xcd * per + local;
  return tall * per + (xcd - tall) * (per - 1) + local;
}

// Grouped ("super-row") tile order of the reference GEMM: consecutive ids walk GROUP_M tiles
// down before stepping one tile right (python/tutorials/03-matrix-multiplication.py:265-273).
__device__ __forceinline__ void grouped_tile(int pid, int num_m, int num_n, int group_m, int& pm, int& pn) {
  int in_group = group_m * num_n;
  int gid = pid / in_group;
  int first = gid * group_m;
  int gsz = min(num_m - first, group_m);
  pm = first + (pid % in_group) % gsz;
  pn = (pid % in_group) / gsz;
}

}  // namespace mi355

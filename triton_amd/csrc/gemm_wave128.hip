// Four-wave GEMM with 128x128 of C per wave, built from 16x16x32 MFMAs (K-major A and B, 16-bit
// types): one workgroup per 256x256 tile of C, one wave per SIMD, all 256 accumulator registers of
// a lane in use.
//
// Why this shape: the GEMM runs at the board's power limit, and on N(0,1) operands a stream of
// 16x16x32 MFMAs needs 11 % less energy per flop than a stream of 32x32x16 ones (16.9 vs 19.1 ns per
// 32768 flop and SIMD, measured with nothing else running).  Against the eight-wave kernels of
// gemm_core.h (128x64 per wave) every flop also needs a third fewer LDS fragment bytes.
//
// Loop: 128 bytes of every operand row per K step (two sub-steps of 64 MFMAs), two 64 KiB LDS
// stages filled by direct global->LDS loads.  With a single wave per SIMD nothing else can issue
// MFMAs while that wave is held up, so the memory instructions carry no scalar arithmetic: the
// sixteen scalar bases of a wave's loads are fixed, the K position travels in the lane offset,
// and the eight loads of one operand share one M0 value through their instruction offsets (which
// the hardware adds to the global AND the LDS address).  Every fragment read is issued a sub-step
// before its use.
//
// LDS tile of an operand: row r (128 bytes = eight 16-byte chunks) at r * 128, chunk c in slot
// c ^ ((r >> 1) & 7): the 16 lanes of a ds_read_b128 pass (16 consecutive rows, one chunk) cover
// all 64 banks once.  The direct loads write LDS linearly (lane i -> base + 16 i), so the
// permutation is applied to the global address each lane fetches.
#include "gemm_core.h"

namespace mi355 {

// D(16x16 fp32) += A(16x32) * B(32x16).  Lane l supplies A[l%16][8*(l/16) .. +8] and
// B[8*(l/16) .. +8][l%16]; accumulator register r of lane l is D[4*(l/16) + r][l%16].
// Issued as inline assembly with the accumulator constrained to the accumulation registers: left to
// the register allocator, some of the 64 accumulator tuples of a lane end up in architectural
// registers and get shuffled back and forth in every K step.
__device__ __forceinline__ void mfma16(bf16x8 a, bf16x8 b, f32x4& c) {
#if MI355_DEVICE_PASS
  asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
#endif
}
__device__ __forceinline__ void mfma16(f16x8 a, f16x8 b, f32x4& c) {
#if MI355_DEVICE_PASS
  asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
#endif
}

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
static int wave128_grid(int tiles, int cap) {
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

// The tiles `tile`, `tile + tile_step`, ... (< `tile_stop`, by default M/256 * N/256) of one problem, computed by the calling workgroup
// with the 128 KiB of LDS at `lds0`.  XCD: pass the tile numbers through the per-XCD remap first.  EPI: 0 = scales,
// activation, any output type; 1 = C has the type of the operands, no scales, no activation; 2 = 0 plus the addend.
template <typename V8, bool B_KMAJOR, bool XCD, int EPI = 0>
__device__ __forceinline__ void gemm_wave128_tiles(const GemmArgs& p, int tile, const int tile_step, const unsigned lds0, const int tile_stop = -1) {
#if MI355_DEVICE_PASS
  constexpr int BM = 256, BN = 256, ROWB = 128;
  constexpr int A_BYTES = BM * ROWB, STAGE = A_BYTES + BN * ROWB;  // 64 KiB
  constexpr int MT = 8, NT = 8, KS = 2;                             // 16x16 tiles per wave, 16x16x32 sub-steps per stage
  constexpr int NM = MT * NT;                                       // MFMAs per sub-step

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int l16 = lane & 15, kg = lane >> 4;

  const int num_m = p.M / BM, num_n = p.N / BN;
  const int ntiles = num_m * num_n;
  const int tend = tile_stop < 0 ? ntiles : tile_stop;   // the walk ends before this tile
  // The tiles are computed as ONE stream of K steps: the loads of the last two steps of a tile already
  // fetch the first two K steps of the next one, so its first fragments are in registers when the finished
  // tile is stored.
  auto tile_at = [&](int t, int& tm, int& tn) { grouped_tile(XCD ? xcd_remap(t, ntiles) : t, num_m, num_n, p.group_m, tm, tn); };
  int pm, pn;
  tile_at(tile, pm, pn);
  const int nk = p.k_bytes / ROWB;
  int nk_last = nk;   // the same number, but opaque: see mfma_retire
  asm volatile("" : "+s"(nk_last));

  // ---- direct loads: instruction q = 8 * wave + j moves rows 8 q .. 8 q + 7 of a tile; the swizzle of
  // those rows is 4 (q & 1) + lane / 16, so the lane offset depends on the parity of j only
  const unsigned drow = lane >> 3, dslot = lane & 7;
  unsigned voffA[2], voffB[B_KMAJOR ? 2 : 1];
#pragma unroll
  for (int par = 0; par < 2; par++) {
    const unsigned chunk = dslot ^ ((par * 4 + (lane >> 4)) & 7);
    voffA[par] = drow * (unsigned)p.lda + chunk * 16;
    if constexpr (B_KMAJOR) voffB[par] = drow * (unsigned)p.ldb + chunk * 16;
  }
  // Row-major B[K, N]: the stage holds 64 k rows of 512 bytes; instruction q = 8 * wave + j moves the k rows
  // 2 q, 2 q + 1 (lane i: row i / 32, physical 16-byte chunk i % 32).  Element (k, n) lives in the 32-byte
  // column group (n / 16) ^ 2 (k & 3) ^ ((k >> 3) & 1) of its row: a transpose read is served two 16-lane
  // groups at a time - four consecutive k rows each, eight rows apart, the same 16 columns - and this
  // spreads those 8 x 32 bytes over all banks.  With k = 16 wave + 2 j + i / 32 the XOR terms are
  // 4 (j & 1) + 2 (i / 32) and (j >> 2) & 1: the j terms are XORed into the lane offset at each load.
  if constexpr (!B_KMAJOR) {
    const unsigned pg = (lane & 31) >> 1, half = lane & 1;
    // j = 0; other j: XOR below (which needs a pitch that is a multiple of 512 bytes)
    voffB[0] = (lane >> 5) * (unsigned)p.ldb + ((pg ^ (2 * (lane >> 5))) * 32) + half * 16;
  }
  // scalar bases of the tile the loads are fetching (two K steps ahead of the MFMAs)
  const char* gA;
  const char* gB;
  auto set_fill_tile = [&](int fm, int fn) {
    gA = p.A + ((int64_t)fm * BM + wave * 64) * p.lda;
    gB = B_KMAJOR ? p.B + ((int64_t)fn * BN + wave * 64) * p.ldb
                  : p.B + (int64_t)fn * BN * 2 + (int64_t)(wave * 16) * p.ldb;
  };
  set_fill_tile(pm, pn);
  const int64_t stepA = 8 * p.lda, stepB = (B_KMAJOR ? 8 : 2) * p.ldb;
  const unsigned kstepB = B_KMAJOR ? ROWB : 64 * (unsigned)p.ldb;   // bytes from one K step to the next
  // load j (0..7: A, 8..15: B) of tile kt into the stage at `stage_base`.  M0 = middle of the wave's
  // 8 KiB of that operand, instruction offsets -4096 .. 3072 (taken back out of the scalar base).
  auto issue = [&](auto J_, int kt, unsigned stage_base) {
    constexpr int j = decltype(J_)::value, q = j & 7, ioff = (q - 4) * 1024;
    const char* src = (j < 8 ? gA + q * stepA : gB + q * stepB) - ioff;
    const unsigned dst = stage_base + (j < 8 ? 0 : A_BYTES) + wave * 8192 + 4096;
    unsigned lane_off;
    if constexpr (j < 8) lane_off = voffA[j & 1] + (unsigned)kt * ROWB;
    else if constexpr (B_KMAJOR) lane_off = voffB[j & 1] + (unsigned)kt * ROWB;
    else lane_off = (voffB[0] ^ ((4 * (q & 1) + ((q >> 2) & 1)) * 32)) + (unsigned)kt * kstepB;
    async_copy16_sbase_off<ioff, q == 0>(src, lane_off, dst);
  };

  // ---- fragment reads: lane (l16, kg) of sub-step ks wants chunk 4 ks + kg of row l16 (+ 16 t)
  unsigned adrA[KS], adrB[B_KMAJOR ? KS : NT];   // stage 0; stage 1 is 64 KiB further (added at the read)
  {
    const unsigned s = (l16 >> 1) & 7;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      const unsigned slot = ((4 * ks + kg) ^ s) * 16;
      adrA[ks] = lds0 + (wm * 128 + l16) * ROWB + slot;
      if constexpr (B_KMAJOR) adrB[ks] = lds0 + A_BYTES + (wn * 128 + l16) * ROWB + slot;
    }
    // row-major B: lane i of the 16-lane group kg addresses k row 8 kg + i / 4 (+ 32 ks, + 4 for the second
    // read) and the 8 bytes (i & 3) of the 16-column group of tile t; (k & 3) = i / 4 and (k >> 3) & 1 = kg & 1
    // for every ks and both reads
    if constexpr (!B_KMAJOR) {
      const unsigned k = 8 * kg + (l16 >> 2), m = (2 * (l16 >> 2)) ^ (kg & 1);
#pragma unroll
      for (int t = 0; t < NT; t++) adrB[t] = lds0 + A_BYTES + k * (BN * 2) + ((wn * 8 + (t ^ m)) * 32) + (l16 & 3) * 8;
    }
  }
  static_assert(STAGE == 65536, "stage 1 = stage 0 + 64 KiB");
  struct Frags { V8 a[MT]; V8 b[NT]; };
  Frags f[2];
  constexpr int NRD = MT + NT;  // fragment reads per sub-step (a row-major B fragment takes two instructions)
  auto read_one = [&](auto OP_, auto P_, auto KS_, Frags& dst) {
    constexpr int op = decltype(OP_)::value, P = decltype(P_)::value, ks = decltype(KS_)::value;
    constexpr unsigned so = P * STAGE;
    if constexpr (op < MT) {
      dst.a[op] = __builtin_bit_cast(V8, lds_read_b128<op * 16 * ROWB>(adrA[ks] + so));
    } else if constexpr (B_KMAJOR) {
      dst.b[op - MT] = __builtin_bit_cast(V8, lds_read_b128<(op - MT) * 16 * ROWB>(adrB[ks] + so));
    } else {
      // two transpose reads per fragment: k .. k + 3 into the low, k + 4 .. k + 7 into the high half
      constexpr int t = op - MT, imm = ks * 32 * BN * 2;
      // (the compiler's own builtin, not inline assembly: it can then place the two halves directly in
      // the four-register operand; its wait-count bookkeeping only ever adds to the explicit waits)
      const unsigned ad = adrB[t] + so + imm;
      s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_PTR(s16x4))(uintptr_t)ad);
      s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_PTR(s16x4))(uintptr_t)(ad + 4 * BN * 2));
      dst.b[t] = __builtin_bit_cast(V8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
    }
  };
  auto pin = [&](Frags& x) {
    static_for<MT>([&](auto T_) { lds_use(x.a[decltype(T_)::value]); });
    static_for<NT>([&](auto T_) { lds_use(x.b[decltype(T_)::value]); });
  };

  f32x4 acc[MT][NT];
  auto zero_acc = [&]() {
#pragma unroll
    for (int i = 0; i < MT; i++)
#pragma unroll
      for (int j = 0; j < NT; j++) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  };
  zero_acc();

  // ---- prologue: both stages requested, first fragments of stage 0 read
  static_for<16>([&](auto J_) { issue(J_, 0, lds0); });
  static_for<16>([&](auto J_) { issue(J_, 1, lds0 + STAGE); });
  wait_vmcnt<16>();
  block_barrier();
  using Z = std::integral_constant<int, 0>;
  static_for<NRD>([&](auto OP_) { read_one(OP_, Z{}, Z{}, f[0]); });

  // One sub-step: 64 MFMAs on f[ks]; the fragments of the next sub-step are requested over the first
  // half of them (one read per two MFMAs).  The last sub-step of a stage first meets the other waves
  // (every wave has then read all it needs of this stage, and the other stage has landed), reads the
  // first fragments of the other stage and refills this one with the tile two steps ahead (one load
  // per four MFMAs).
  auto substep = [&](auto P_, auto KS_, auto MORE_, auto REFILL_, int kt) {
    constexpr int P = decltype(P_)::value, ks = decltype(KS_)::value, cur = ks & 1, nxt = cur ^ 1;
    constexpr bool last = ks == KS - 1;
    constexpr bool more = decltype(MORE_)::value;              // there is a next sub-step to read for
    constexpr bool refill = last && decltype(REFILL_)::value;  // and a tile two steps ahead to request
    lds_wait<0>();
    pin(f[cur]);
    if constexpr (last) {
      wait_vmcnt<0>();
      block_barrier();
    }
    static_for<NM>([&](auto N_) {
      constexpr int n = decltype(N_)::value, i = n / NT, j = n % NT;
      mfma16(f[cur].b[j], f[cur].a[i], acc[i][j]);
      // one fragment read per two MFMAs over the first half, one direct load per four MFMAs (64 cycles) over the
      // whole sub-step: loads issued faster than the memory pipeline takes them hold up the MFMAs behind them
      // (one per two MFMAs: -3.5 %)
      if constexpr (more && n % 2 == 0 && n / 2 < NRD)
        read_one(std::integral_constant<int, n / 2>{}, std::integral_constant<int, last ? (P ^ 1) : P>{},
                 std::integral_constant<int, last ? 0 : ks + 1>{}, f[nxt]);
      if constexpr (refill && n % 4 == 1) issue(std::integral_constant<int, n / 4>{}, kt + 2, lds0 + P * STAGE);
      if constexpr (n % 2 == 1) __builtin_amdgcn_sched_barrier(0);
    });
  };
  using I0 = std::integral_constant<int, 0>; using I1 = std::integral_constant<int, 1>;
  using T = std::true_type; using F = std::false_type;
  // A K step: `fk` is the K step (of the tile the scalar bases point at) that its loads fetch.
  auto stage = [&](auto P_, int fk) {
    substep(P_, I0{}, T{}, F{}, fk - 2);
    substep(P_, I1{}, T{}, T{}, fk - 2);
    // The fragment reads above are invisible to the compiler: have them landed before control reaches a loop
    // edge, where the register allocator may copy the registers they write.  (They were issued over the first
    // half of the sub-step, so this does not wait.)
    lds_wait<0>();
    pin(f[0]);
  };
  // The fill cursor runs two K steps ahead of the MFMAs, across tile boundaries; behind the last tile it
  // wraps to that tile's first steps again (fetched into stages nobody reads any more), which keeps the
  // loop, the number of loads in flight and every wait uniform.
  int fk = 2, ftile = tile;   // next K step to fetch, and the tile it belongs to
  auto advance = [&]() {
    if (++fk == nk) {
      fk = 0;
      if (ftile + tile_step < tend) {
        ftile += tile_step;
        int fm, fn;
        tile_at(ftile, fm, fn);
        set_fill_tile(fm, fn);
      }
    }
  };
  if (nk == 2) { fk = 1; advance(); }   // (two steps per tile: the prologue fetched both, the cursor is on the next tile)
  while (true) {
    for (int kt = 0; kt < nk; kt += 2) {
      stage(I0{}, fk); advance();
      stage(I1{}, fk); advance();
      if (kt + 2 >= nk_last) mfma_retire();
    }
    // The next tile's first fragments were requested by reads the compiler cannot see: have them landed
    // before the epilogue's register traffic could move their registers.  Nor does it know that the assembly
    // above are MFMAs: let the last ones retire before their results are read.
    lds_wait<0>();
    pin(f[0]);
    mfma_drain(acc);
    // (the tile and lane coordinates pass through an empty assembly statement so that none of the
    // epilogue's address arithmetic is hoisted out of the tile loop, where it would occupy - and spill -
    // registers throughout the K loop)
    int em = pm * BM + wm * 128, en = pn * BN + wn * 128, el = l16, ek = kg;
    asm volatile("" : "+s"(em), "+s"(en), "+v"(el), "+v"(ek));
    if constexpr (EPI == 1) gemm_epilogue16_plain<MT, NT, std::conditional_t<std::is_same<V8, bf16x8>::value, __bf16, _Float16>>(acc, p, em, en, el, ek);
    else gemm_epilogue16<MT, NT, EPI == 2>(acc, p, em, en, el, ek);
    tile += tile_step;
    if (tile >= tend) break;
    tile_at(tile, pm, pn);
    zero_acc();
  }
  wait_vmcnt<0>();  // nothing may still be writing LDS when the workgroup ends
#endif
}

// Workgroup b computes the tiles b, b + gridDim.x, ... (the grid: wave128_grid).
template <typename V8, bool B_KMAJOR, bool AUX>
__global__ __launch_bounds__(256, 1) void gemm_wave128_kernel(GemmArgs p) {
#if MI355_DEVICE_PASS
  extern __shared__ __attribute__((aligned(1024))) char lds_raw[];
  gemm_wave128_tiles<V8, B_KMAJOR, true, AUX ? 2 : 0>(p, blockIdx.x, gridDim.x, lds_addr((LDS_PTR(const void))lds_raw));
#endif
}

// Grouped GEMM (python/tutorials/08-grouped-gemm.py:64-140: pointers, sizes and leading dimensions of the
// problems in device arrays, row-major B) for groups made of whole 256x256 tiles: gridDim.x workgroups walk
// the tiles of all problems, numbered problem after problem; a tile is one run of the stream above (its
// loads wrap around to the tile's own first steps at the end), so consecutive tiles of a workgroup may
// belong to different problems.  Every workgroup first reads the tables and returns unless this kernel is
// the one that the group's shapes select (grouped_plan).
template <typename V8>
__global__ __launch_bounds__(256, 1) void gemm_wave128_grouped_kernel(GroupedArgs ga) {
#if MI355_DEVICE_PASS
  extern __shared__ __attribute__((aligned(1024))) char lds_raw[];
  const unsigned lds0 = lds_addr((LDS_PTR(const void))lds_raw);
  long long total = 0;
  if (grouped_plan(ga, &total) != 2) return;
  // The tiles of all problems, numbered problem after problem, are dealt in chunks of c consecutive tiles:
  // program w (renumbered so that the programs of one XCD are neighbours) takes the chunks w, w + nprog, ...
  // The part of a chunk inside one problem is one stream of K steps (tile after tile down a column of C
  // tiles: the B panel is fetched once); the stream restarts at the next chunk and where a chunk crosses into
  // the next problem.  c = tiles per program, at most `chunk` (4): longer runs save more restarts, but all
  // programs together then work on nprog * c tiles at a time, and with 256 programs on 2048^3 problems eight
  // tiles each already spread over 32 problems, more operands than the last-level cache holds (-8 % there,
  // against +8 to +17 % for four tiles each on 16 such problems).
  const int nprog = gridDim.x;
  const int w = xcd_remap(blockIdx.x, nprog);
  const int tot = (int)total;
  const int c = max(1, min(ga.chunk, (tot + nprog - 1) / nprog));
  int chunk = w;
  int cur = chunk * c, limit = min(cur + c, tot);
  int first = 0;   // number of the first tile of problem gi
  for (int gi = 0; gi < ga.group_size && cur < tot; gi++) {
    const int gm = ga.sizes[gi * 3], gn = ga.sizes[gi * 3 + 1], gk = ga.sizes[gi * 3 + 2];
    const int num_tiles = (gm / 256) * (gn / 256);
    if (cur < first + num_tiles) {
      const int ldc = ga.lds[gi * 3 + 2];
      GemmArgs p{};
      p.A = (const char*)ga.a_ptrs[gi]; p.B = (const char*)ga.b_ptrs[gi]; p.C = (char*)ga.c_ptrs[gi];
      p.M = gm; p.N = gn; p.K = gk; p.k_bytes = gk * 2;
      p.lda = (int64_t)ga.lds[gi * 3] * 2; p.ldb = (int64_t)ga.lds[gi * 3 + 1] * 2; p.ldc = ldc; p.scn = 1;
      p.out_dtype = ga.out_dtype; p.group_m = 8;
      p.c_vec_ok = (ldc % 4 == 0) && (((uintptr_t)p.C) % 16 == 0);
      while (cur < tot && cur < first + num_tiles) {
        const int stop = min(limit, first + num_tiles) - first;
        gemm_wave128_tiles<V8, false, false, 1>(p, cur - first, 1, lds0, stop);
        block_barrier();   // the next run's loads overwrite the stages: every wave must be done reading them
        cur = first + stop;
        if (cur == limit) {
          chunk += nprog;
          cur = chunk * c;
          limit = min(cur + c, tot);
        }
      }
    }
    first += num_tiles;
  }
#endif
}

// ---------------------------------------------------------------------------------------------
// The same kernel for fp8 (e4m3fn / e5m2, both operands K-major): 16x16x128 f8f6f4 MFMAs, one per
// accumulator tile and K step (128 bytes of K = one whole LDS row).  A fragment is 32 bytes per
// lane (two 16-byte chunks, eight registers), so a K step's sixteen fragments fill 128 registers;
// the step is split in two halves by rows of A: the first uses A fragments 0..3, the second 4..7
// (read during the first), while the B fragments and the first four A fragments of the next
// stage are read during the second half into a second set.  Any assignment of K positions to the
// bytes of a lane works as long as A and B use the same one: lane (r, kg) takes the chunks
// 2 kg and 2 kg + 1 of its row.  The fragment reads are ordinary LDS loads here (the compiler then
// places the two halves directly in the eight-register operand and waits for each fragment just
// before its first use); the direct global->LDS loads stay invisible to its bookkeeping.
// ---------------------------------------------------------------------------------------------
template <int FMT>
__device__ __forceinline__ void mfma16_f8(const i32x8& a, const i32x8& b, f32x4& c) {
#if MI355_DEVICE_PASS
  if constexpr (FMT == 0) asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
  else asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, %0 cbsz:1 blgp:1" : "+a"(c) : "v"(a), "v"(b));
#endif
}

template <int FMT, bool AUX>
__global__ __launch_bounds__(256, 1) void gemm_wave128_f8_kernel(GemmArgs p) {
#if MI355_DEVICE_PASS
  constexpr int BM = 256, BN = 256, ROWB = 128;
  constexpr int A_BYTES = BM * ROWB, STAGE = A_BYTES + BN * ROWB;  // 64 KiB
  constexpr int MT = 8, NT = 8, MH = MT / 2;
  extern __shared__ __attribute__((aligned(1024))) char lds_raw[];
  const unsigned lds0 = lds_addr((LDS_PTR(const void))lds_raw);

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int l16 = lane & 15, kg = lane >> 4;

  const int num_m = p.M / BM, num_n = p.N / BN;
  const int ntiles = num_m * num_n;
  int tile = blockIdx.x;   // this workgroup computes the tiles tile, tile + gridDim.x, ... as one stream of K steps
  int pm, pn;
  grouped_tile(xcd_remap(tile, ntiles), num_m, num_n, p.group_m, pm, pn);
  const int nk = p.k_bytes / ROWB;
  int nk_last = nk;   // the same number, but opaque: see mfma_retire
  asm volatile("" : "+s"(nk_last));

  // ---- direct loads, exactly as in the 16-bit kernel (the tiles are the same bytes)
  const unsigned drow = lane >> 3, dslot = lane & 7;
  unsigned voffA[2], voffB[2];
#pragma unroll
  for (int par = 0; par < 2; par++) {
    const unsigned chunk = dslot ^ ((par * 4 + (lane >> 4)) & 7);
    voffA[par] = drow * (unsigned)p.lda + chunk * 16;
    voffB[par] = drow * (unsigned)p.ldb + chunk * 16;
  }
  // scalar bases of the tile the loads are fetching (two K steps ahead of the MFMAs)
  const char* gA;
  const char* gB;
  auto set_fill_tile = [&](int fm, int fn) {
    gA = p.A + ((int64_t)fm * BM + wave * 64) * p.lda;
    gB = p.B + ((int64_t)fn * BN + wave * 64) * p.ldb;
  };
  set_fill_tile(pm, pn);
  const int64_t stepA = 8 * p.lda, stepB = 8 * p.ldb;
  auto issue = [&](auto J_, int kt, unsigned stage_base) {
    constexpr int j = decltype(J_)::value, q = j & 7, ioff = (q - 4) * 1024;
    const char* src = (j < 8 ? gA + q * stepA : gB + q * stepB) - ioff;
    const unsigned dst = stage_base + (j < 8 ? 0 : A_BYTES) + wave * 8192 + 4096;
    const unsigned lane_off = (j < 8 ? voffA[j & 1] : voffB[j & 1]) + (unsigned)kt * ROWB;
    async_copy16_sbase_off<ioff, q == 0>(src, lane_off, dst);
  };

  // ---- fragment reads: lane (l16, kg) wants the chunks 2 kg, 2 kg + 1 of row l16 (+ 16 t)
  LDS_PTR(const char) fragA[2];
  LDS_PTR(const char) fragB[2];
  {
    const unsigned s = (l16 >> 1) & 7;
#pragma unroll
    for (int c = 0; c < 2; c++) {
      const unsigned slot = ((2 * kg + c) ^ s) * 16;
      fragA[c] = (LDS_PTR(const char))lds_raw + (wm * 128 + l16) * ROWB + slot;
      fragB[c] = (LDS_PTR(const char))lds_raw + A_BYTES + (wn * 128 + l16) * ROWB + slot;
    }
  }
  auto read_frag = [&](LDS_PTR(const char) (&base)[2], int off) {
    i32x4 lo = *(LDS_PTR(const i32x4))(base[0] + off);
    i32x4 hi = *(LDS_PTR(const i32x4))(base[1] + off);
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  };
  i32x8 a0[MH], a1[MH], b[2][NT];

  f32x4 acc[MT][NT];
  auto zero_acc = [&]() {
#pragma unroll
    for (int i = 0; i < MT; i++)
#pragma unroll
      for (int j = 0; j < NT; j++) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  };
  zero_acc();

  // ---- prologue: both stages requested, B and the first four A fragments of stage 0 read
  static_for<16>([&](auto J_) { issue(J_, 0, lds0); });
  static_for<16>([&](auto J_) { issue(J_, 1, lds0 + STAGE); });
  wait_vmcnt<16>();
  block_barrier();
#pragma unroll
  for (int t = 0; t < NT; t++) b[0][t] = read_frag(fragB, t * 16 * ROWB);
#pragma unroll
  for (int t = 0; t < MH; t++) a0[t] = read_frag(fragA, t * 16 * ROWB);

  // One K step on stage P with the B fragments of set `cur`; its loads fetch K step `fk` of the fill tile.
  auto step = [&](auto P_, auto CUR_, int fk) {
    constexpr int P = decltype(P_)::value, cur = decltype(CUR_)::value, nxt = cur ^ 1;
    constexpr int so = P * STAGE, sn = (P ^ 1) * STAGE;
    // first half: rows 0..3 of A; the A fragments 4..7 of this stage are read meanwhile
    static_for<MH * NT>([&](auto N_) {
      constexpr int n = decltype(N_)::value, i = n / NT, j = n % NT;
      mfma16_f8<FMT>(b[cur][j], a0[i], acc[i][j]);
      if constexpr (n % 4 == 0 && n / 4 < MH) a1[n / 4] = read_frag(fragA, so + (MH + n / 4) * 16 * ROWB);
      if constexpr (n % 2 == 1) __builtin_amdgcn_sched_barrier(0);
    });
    // every wave has now requested all it needs of stage P: once those reads are back and the other
    // stage has landed, meet, then read the next fragments from the other stage and refill this one
    lds_wait<0>();
    wait_vmcnt<0>();
    block_barrier();
    static_for<MH * NT>([&](auto N_) {
      constexpr int n = decltype(N_)::value, i = n / NT, j = n % NT;
      mfma16_f8<FMT>(b[cur][j], a1[i], acc[MH + i][j]);
      if constexpr (n < NT) b[nxt][n] = read_frag(fragB, sn + n * 16 * ROWB);
      if constexpr (n >= NT && n < NT + MH) a0[n - NT] = read_frag(fragA, sn + (n - NT) * 16 * ROWB);
      if constexpr (n % 2 == 1) issue(std::integral_constant<int, n / 2>{}, fk, lds0 + P * STAGE);
      if constexpr (n % 2 == 1) __builtin_amdgcn_sched_barrier(0);
    });
  };
  using I0 = std::integral_constant<int, 0>; using I1 = std::integral_constant<int, 1>;
  // The fill cursor runs two K steps ahead of the MFMAs, across tile boundaries; behind the last tile it
  // wraps to that tile's first steps again (fetched into stages nobody reads any more), which keeps the
  // loop, the number of loads in flight and every wait uniform.
  int fk = 2, ftile = tile;
  auto advance = [&]() {
    if (++fk == nk) {
      fk = 0;
      if (ftile + (int)gridDim.x < ntiles) {
        ftile += gridDim.x;
        int fm, fn;
        grouped_tile(xcd_remap(ftile, ntiles), num_m, num_n, p.group_m, fm, fn);
        set_fill_tile(fm, fn);
      }
    }
  };
  if (nk == 2) { fk = 1; advance(); }
  while (true) {
    for (int kt = 0; kt < nk; kt += 2) {
      step(I0{}, I0{}, fk); advance();
      step(I1{}, I1{}, fk); advance();
      if (kt + 2 >= nk_last) mfma_retire();
    }
    mfma_drain(acc);
    int em = pm * BM + wm * 128, en = pn * BN + wn * 128, el = l16, ek = kg;
    asm volatile("" : "+s"(em), "+s"(en), "+v"(el), "+v"(ek));   // (keeps the epilogue's address arithmetic out of the K loop)
    gemm_epilogue16<MT, NT, AUX>(acc, p, em, en, el, ek);
    tile += gridDim.x;
    if (tile >= ntiles) break;
    grouped_tile(xcd_remap(tile, ntiles), num_m, num_n, p.group_m, pm, pn);
    zero_acc();
  }
  wait_vmcnt<0>();  // nothing may still be writing LDS when the workgroup ends
#endif
}

// Scaled fp8 (e4m3) MFMA with the accumulator pinned to the accumulation registers; byte 0 of the scale dwords.
__device__ __forceinline__ void mfma16_mxfp8(const i32x8& a, const i32x8& b, f32x4& c, int sa, int sb) {
#if MI355_DEVICE_PASS
  asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel_hi:[0,0,0]"
               : "+a"(c) : "v"(a), "v"(b), "v"(sa), "v"(sb));
#endif
}
#ifndef MXFP8_CHUNK
#define MXFP8_CHUNK(kg, c) ((kg) + 4 * (c))
#endif

// MXFP8 (e4m3 codes, one e8m0 scale per 32 elements): the fp8 kernel above with scaled MFMAs; a K step is
// 128 elements = four scale blocks, the scales travel 16 bytes per row (four K steps) per direct load into a
// two-slot LDS ring like those of the MXFP4 kernel below.
__global__ __launch_bounds__(256, 1) void gemm_wave128_mxfp8_kernel(GemmArgs p) {
#if MI355_DEVICE_PASS
  constexpr int BM = 256, BN = 256, ROWB = 128;
  constexpr int A_BYTES = BM * ROWB, STAGE = A_BYTES + BN * ROWB;  // 64 KiB
  constexpr int MT = 8, NT = 8, MH = MT / 2;
  constexpr int SC_BASE = 2 * STAGE, SC_SLOT = (BM + BN) * 16;      // scale ring behind the two stages
  extern __shared__ __attribute__((aligned(1024))) char lds_raw[];
  const unsigned lds0 = lds_addr((LDS_PTR(const void))lds_raw);

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int l16 = lane & 15, kg = lane >> 4;

  const int num_m = p.M / BM, num_n = p.N / BN;
  const int ntiles = num_m * num_n;
  int tile = blockIdx.x;   // this workgroup computes the tiles tile, tile + gridDim.x, ... as one stream of K steps
  int pm, pn;
  grouped_tile(xcd_remap(tile, ntiles), num_m, num_n, p.group_m, pm, pn);
  const int nk = p.k_bytes / ROWB;
  int nk_last = nk;   // the same number, but opaque: see mfma_retire
  asm volatile("" : "+s"(nk_last));

  // ---- direct loads, exactly as in the 16-bit kernel (the tiles are the same bytes)
  const unsigned drow = lane >> 3, dslot = lane & 7;
  unsigned voffA[2], voffB[2];
#pragma unroll
  for (int par = 0; par < 2; par++) {
    const unsigned chunk = dslot ^ ((par * 4 + (lane >> 4)) & 7);
    voffA[par] = drow * (unsigned)p.lda + chunk * 16;
    voffB[par] = drow * (unsigned)p.ldb + chunk * 16;
  }
  // scalar bases of the tile the loads are fetching (two K steps ahead of the MFMAs)
  const char* gA;
  const char* gB;
  const char* gSA;
  const char* gSB;
  auto set_fill_tile = [&](int fm, int fn) {
    gA = p.A + ((int64_t)fm * BM + wave * 64) * p.lda;
    gB = p.B + ((int64_t)fn * BN + wave * 64) * p.ldb;
    gSA = (const char*)p.sA + ((int64_t)fm * BM + wave * 64) * p.lds_a;
    gSB = (const char*)p.sB + ((int64_t)fn * BN + wave * 64) * p.lds_b;
  };
  set_fill_tile(pm, pn);
  const int64_t stepA = 8 * p.lda, stepB = 8 * p.ldb;
  auto issue = [&](auto J_, int kt, unsigned stage_base) {
    constexpr int j = decltype(J_)::value, q = j & 7, ioff = (q - 4) * 1024;
    const char* src = (j < 8 ? gA + q * stepA : gB + q * stepB) - ioff;
    const unsigned dst = stage_base + (j < 8 ? 0 : A_BYTES) + wave * 8192 + 4096;
    const unsigned lane_off = (j < 8 ? voffA[j & 1] : voffB[j & 1]) + (unsigned)kt * ROWB;
    async_copy16_sbase_off<ioff, q == 0>(src, lane_off, dst);
  };

  // ---- scale loads: wave w fetches the 16 scale bytes (four K steps) of rows 64 w .. 64 w + 63 of A and of B
  const unsigned voffSA = lane * (unsigned)p.lds_a, voffSB = lane * (unsigned)p.lds_b;
  auto issue_scales = [&](int g) {   // group g of four K steps of the fill tile -> slot g & 1 (K steps come in eights)
    const unsigned slot = lds0 + SC_BASE + (g & 1) * SC_SLOT + wave * 1024;
    async_copy16_sbase(gSA, voffSA + (unsigned)g * 16, slot);
    async_copy16_sbase(gSB, voffSB + (unsigned)g * 16, slot + BM * 16);
  };
  // scales of a K step: the dword of the step's four blocks, shifted so that this lane group's byte is byte 0
  const unsigned adrSA = lds0 + SC_BASE + (wm * 128 + l16) * 16;
  const unsigned adrSB = lds0 + SC_BASE + BM * 16 + (wn * 128 + l16) * 16;
  const int sshift = 8 * kg;
  int sa[2][MT], sb[2][NT];
  auto read_scales = [&](auto SET_, auto OFF_) {   // OFF: slot * SC_SLOT + (K step & 3) * 4
    constexpr int set = decltype(SET_)::value, off = decltype(OFF_)::value;
    static_for<MT>([&](auto T_) { constexpr int t = decltype(T_)::value; sa[set][t] = lds_read_b32<off + t * 256>(adrSA); });
    static_for<NT>([&](auto T_) { constexpr int t = decltype(T_)::value; sb[set][t] = lds_read_b32<off + t * 256>(adrSB); });
  };
  auto fix_scales = [&](auto SET_) {
    constexpr int set = decltype(SET_)::value;
    static_for<MT>([&](auto T_) { constexpr int t = decltype(T_)::value; lds_use(sa[set][t]); sa[set][t] = (int)((unsigned)sa[set][t] >> sshift); });
    static_for<NT>([&](auto T_) { constexpr int t = decltype(T_)::value; lds_use(sb[set][t]); sb[set][t] = (int)((unsigned)sb[set][t] >> sshift); });
  };

  // ---- fragment reads.  The 8-bit forms of the scaled MFMA split a lane's 32 bytes: registers 0-3 of the lane
  // groups 2 b, 2 b + 1 together are scale block b, registers 4-7 block 2 + b, and block b takes its scale from
  // lane group b.  So lane (l16, kg) reads chunk kg into its low and chunk 4 + kg into its high registers and
  // supplies the scale of block kg.
  LDS_PTR(const char) fragA[2];
  LDS_PTR(const char) fragB[2];
  {
    const unsigned s = (l16 >> 1) & 7;
#pragma unroll
    for (int c = 0; c < 2; c++) {
      const unsigned slot = ((MXFP8_CHUNK(kg, c)) ^ s) * 16;
      fragA[c] = (LDS_PTR(const char))lds_raw + (wm * 128 + l16) * ROWB + slot;
      fragB[c] = (LDS_PTR(const char))lds_raw + A_BYTES + (wn * 128 + l16) * ROWB + slot;
    }
  }
  auto read_frag = [&](LDS_PTR(const char) (&base)[2], int off) {
    i32x4 lo = *(LDS_PTR(const i32x4))(base[0] + off);
    i32x4 hi = *(LDS_PTR(const i32x4))(base[1] + off);
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  };
  i32x8 a0[MH], a1[MH], b[2][NT];

  f32x4 acc[MT][NT];
  auto zero_acc = [&]() {
#pragma unroll
    for (int i = 0; i < MT; i++)
#pragma unroll
      for (int j = 0; j < NT; j++) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  };
  zero_acc();

  // ---- prologue: both stages requested, B and the first four A fragments of stage 0 read
  issue_scales(0);
  static_for<16>([&](auto J_) { issue(J_, 0, lds0); });
  static_for<16>([&](auto J_) { issue(J_, 1, lds0 + STAGE); });
  wait_vmcnt<16>();
  block_barrier();
  read_scales(std::integral_constant<int, 0>{}, std::integral_constant<int, 0>{});
  lds_wait<0>();
  fix_scales(std::integral_constant<int, 0>{});
#pragma unroll
  for (int t = 0; t < NT; t++) b[0][t] = read_frag(fragB, t * 16 * ROWB);
#pragma unroll
  for (int t = 0; t < MH; t++) a0[t] = read_frag(fragA, t * 16 * ROWB);

  // K step U (0..7 within a group of eight: stage and register sets U & 1, scale slot U >> 2); its loads fetch
  // K step `fk` of the fill tile.
  auto step = [&](auto U_, int fk) {
    constexpr int U = decltype(U_)::value, P = U & 1, cur = U & 1, nxt = cur ^ 1, UN = (U + 1) & 7;
    constexpr int so = P * STAGE, sn = (P ^ 1) * STAGE;
    static_for<MH * NT>([&](auto N_) {
      constexpr int n = decltype(N_)::value, i = n / NT, j = n % NT;
      mfma16_mxfp8(b[cur][j], a0[i], acc[i][j], sb[cur][j], sa[cur][i]);
      if constexpr (n % 4 == 0 && n / 4 < MH) a1[n / 4] = read_frag(fragA, so + (MH + n / 4) * 16 * ROWB);
      if constexpr (n % 2 == 1) __builtin_amdgcn_sched_barrier(0);
    });
    lds_wait<0>();
    wait_vmcnt<0>();
    block_barrier();
    static_for<MH * NT>([&](auto N_) {
      constexpr int n = decltype(N_)::value, i = n / NT, j = n % NT;
      mfma16_mxfp8(b[cur][j], a1[i], acc[MH + i][j], sb[cur][j], sa[cur][MH + i]);
      if constexpr (n < NT) b[nxt][n] = read_frag(fragB, sn + n * 16 * ROWB);
      if constexpr (n >= NT && n < NT + MH) a0[n - NT] = read_frag(fragA, sn + (n - NT) * 16 * ROWB);
      if constexpr (n == 14) read_scales(std::integral_constant<int, nxt>{}, std::integral_constant<int, (UN >> 2) * SC_SLOT + (UN & 3) * 4>{});
      if constexpr (n % 2 == 1) issue(std::integral_constant<int, n / 2>{}, fk, lds0 + P * STAGE);
      // (the scales of the K steps fk .. fk + 3 are requested in the third step of every four, into the slot whose
      // last reader was the read for the step before this one)
      if constexpr ((U & 3) == 2 && n == 16) issue_scales(fk >> 2);
      if constexpr (n % 2 == 1) __builtin_amdgcn_sched_barrier(0);
    });
    lds_wait<0>();
    fix_scales(std::integral_constant<int, nxt>{});
  };
  using I0 = std::integral_constant<int, 0>; using I1 = std::integral_constant<int, 1>;
  // The fill cursor runs two K steps ahead of the MFMAs, across tile boundaries; behind the last tile it
  // wraps to that tile's first steps again (fetched into stages nobody reads any more), which keeps the
  // loop, the number of loads in flight and every wait uniform.
  int fk = 2, ftile = tile;
  auto advance = [&]() {
    if (++fk == nk) {
      fk = 0;
      if (ftile + (int)gridDim.x < ntiles) {
        ftile += gridDim.x;
        int fm, fn;
        grouped_tile(xcd_remap(ftile, ntiles), num_m, num_n, p.group_m, fm, fn);
        set_fill_tile(fm, fn);
      }
    }
  };
  while (true) {
    for (int kt = 0; kt < nk; kt += 8) {
      static_for<8>([&](auto U_) { step(U_, fk); advance(); });
      if (kt + 8 >= nk_last) mfma_retire();
    }
    mfma_drain(acc);
    int em = pm * BM + wm * 128, en = pn * BN + wn * 128, el = l16, ek = kg;
    asm volatile("" : "+s"(em), "+s"(en), "+v"(el), "+v"(ek));   // (keeps the epilogue's address arithmetic out of the K loop)
    gemm_epilogue16<MT, NT>(acc, p, em, en, el, ek);
    tile += gridDim.x;
    if (tile >= ntiles) break;
    grouped_tile(xcd_remap(tile, ntiles), num_m, num_n, p.group_m, pm, pn);
    zero_acc();
  }
  wait_vmcnt<0>();  // nothing may still be writing LDS when the workgroup ends
#endif
}

bool gemm_wave128_mxfp8_ok(const GemmArgs& p) {
  // whole tiles, K steps in groups of eight (K a multiple of 1024), scale rows that a 16-byte load can fetch
  return p.M % 256 == 0 && p.N % 256 == 0 && p.k_bytes % 1024 == 0 && p.k_bytes >= 1024 &&
         p.lda * 8 + p.k_bytes < (1ll << 31) && p.ldb * 8 + p.k_bytes < (1ll << 31) &&
         p.lds_a % 16 == 0 && p.lds_b % 16 == 0 && ((uintptr_t)p.sA | (uintptr_t)p.sB) % 16 == 0 &&
         p.lds_a * 64 + p.k_bytes / 32 < (1ll << 31) && p.lds_b * 64 + p.k_bytes / 32 < (1ll << 31);
}

int gemm_wave128_mxfp8_launch(const GemmArgs& p, hipStream_t stream) {
  constexpr int smem = 2 * 2 * 256 * 128 + 2 * 512 * 16;
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)gemm_wave128_mxfp8_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) return (int)e;
    attr_set = true;
  }
  const int tiles = (p.M / 256) * (p.N / 256);
  const int grid = wave128_grid(tiles, p.num_programs);
  gemm_wave128_mxfp8_kernel<<<dim3(grid), dim3(256), smem, stream>>>(p);
  return (int)hipGetLastError();
}

template <int FMT, bool AUX>
static int launch_wave128_f8(const GemmArgs& p, hipStream_t stream) {
  constexpr int smem = 2 * 2 * 256 * 128;
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)gemm_wave128_f8_kernel<FMT, AUX>, hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) return (int)e;
    attr_set = true;
  }
  const int tiles = (p.M / 256) * (p.N / 256);
  const int grid = wave128_grid(tiles, p.num_programs);
  gemm_wave128_f8_kernel<FMT, AUX><<<dim3(grid), dim3(256), smem, stream>>>(p);
  return (int)hipGetLastError();
}

int gemm_wave128_f8_launch(const GemmArgs& p, bool e5m2, hipStream_t stream) {
  if (p.aux) return e5m2 ? launch_wave128_f8<1, true>(p, stream) : launch_wave128_f8<0, true>(p, stream);
  return e5m2 ? launch_wave128_f8<1, false>(p, stream) : launch_wave128_f8<0, false>(p, stream);
}

// ---------------------------------------------------------------------------------------------
// MXFP4 (e2m1 codes, one e8m0 scale per 32 elements of K) on the same skeleton: scaled 16x16x128
// f8f6f4 MFMAs, two per accumulator tile and K step (128 bytes of a row = 256 elements = 8 scale
// blocks of 16 bytes).  Lane (r, kg) of sub-step ks multiplies block 2 kg + ks of its row, so the two
// scale bytes a lane needs in a K step are neighbours: shifted down once, the byte selector of the MFMA
// is the compile-time ks.  (Which K positions a lane takes is free as long as A, B and the scales
// agree.)  The scales travel like the operands: 16 bytes per row (two K steps) per direct load into a
// two-slot LDS ring (row r at 16 r), one `ds_read_b32` per fragment and K step from there.
// ---------------------------------------------------------------------------------------------
// Scaled fp4 MFMA with the accumulator pinned to the accumulation registers (see mfma16): byte SEL of the two
// scale dwords applies; fp4 operands are four registers.
template <int SEL>
__device__ __forceinline__ void mfma16_mxfp4(const i32x4& a, const i32x4& b, f32x4& c, int sa, int sb) {
#if MI355_DEVICE_PASS
  if constexpr (SEL == 0)
    asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel_hi:[0,0,0] cbsz:4 blgp:4"
                 : "+a"(c) : "v"(a), "v"(b), "v"(sa), "v"(sb));
  else
    asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel:[1,1,0] op_sel_hi:[0,0,0] cbsz:4 blgp:4"
                 : "+a"(c) : "v"(a), "v"(b), "v"(sa), "v"(sb));
#endif
}

__global__ __launch_bounds__(256, 1) void gemm_wave128_mxfp4_kernel(GemmArgs p) {
#if MI355_DEVICE_PASS
  constexpr int BM = 256, BN = 256, ROWB = 128;
  constexpr int A_BYTES = BM * ROWB, STAGE = A_BYTES + BN * ROWB;  // 64 KiB
  constexpr int SC_BASE = 2 * STAGE, SC_SLOT = (BM + BN) * 16;      // scale ring behind the two stages
  constexpr int MT = 8, NT = 8, KS = 2, NM = MT * NT, NRD = MT + NT;
  extern __shared__ __attribute__((aligned(1024))) char lds_raw[];
  const unsigned lds0 = lds_addr((LDS_PTR(const void))lds_raw);

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int l16 = lane & 15, kg = lane >> 4;

  const int num_m = p.M / BM, num_n = p.N / BN;
  const int ntiles = num_m * num_n;
  int tile = blockIdx.x;   // this workgroup computes the tiles tile, tile + gridDim.x, ... as one stream of K steps
  int pm, pn;
  grouped_tile(xcd_remap(tile, ntiles), num_m, num_n, p.group_m, pm, pn);
  const int nk = p.k_bytes / ROWB;
  int nk_last = nk;   // the same number, but opaque: see mfma_retire
  asm volatile("" : "+s"(nk_last));

  // ---- operand loads, as in the 16-bit kernel
  const unsigned drow = lane >> 3, dslot = lane & 7;
  unsigned voffA[2], voffB[2];
#pragma unroll
  for (int par = 0; par < 2; par++) {
    const unsigned chunk = dslot ^ ((par * 4 + (lane >> 4)) & 7);
    voffA[par] = drow * (unsigned)p.lda + chunk * 16;
    voffB[par] = drow * (unsigned)p.ldb + chunk * 16;
  }
  // scalar bases (operands and scales) of the tile the loads are fetching, two K steps ahead of the MFMAs
  const char* gA;
  const char* gB;
  const char* gSA;
  const char* gSB;
  auto set_fill_tile = [&](int fm, int fn) {
    gA = p.A + ((int64_t)fm * BM + wave * 64) * p.lda;
    gB = p.B + ((int64_t)fn * BN + wave * 64) * p.ldb;
    gSA = (const char*)p.sA + ((int64_t)fm * BM + wave * 64) * p.lds_a;
    gSB = (const char*)p.sB + ((int64_t)fn * BN + wave * 64) * p.lds_b;
  };
  set_fill_tile(pm, pn);
  const int64_t stepA = 8 * p.lda, stepB = 8 * p.ldb;
  auto issue = [&](auto J_, int kt, unsigned stage_base) {
    constexpr int j = decltype(J_)::value, q = j & 7, ioff = (q - 4) * 1024;
    const char* src = (j < 8 ? gA + q * stepA : gB + q * stepB) - ioff;
    const unsigned dst = stage_base + (j < 8 ? 0 : A_BYTES) + wave * 8192 + 4096;
    const unsigned lane_off = (j < 8 ? voffA[j & 1] : voffB[j & 1]) + (unsigned)kt * ROWB;
    async_copy16_sbase_off<ioff, q == 0>(src, lane_off, dst);
  };
  // ---- scale loads: wave w fetches the 16 scale bytes (K steps 2 h, 2 h + 1) of rows 64 w .. 64 w + 63 of A and of B
  const unsigned voffSA = lane * (unsigned)p.lds_a, voffSB = lane * (unsigned)p.lds_b;
  auto issue_scales = [&](int h) {   // pair h of K steps of the fill tile -> slot h & 1 (K steps come in fours, so
    const unsigned slot = lds0 + SC_BASE + (h & 1) * SC_SLOT + wave * 1024;   // the slots alternate across tiles too)
    async_copy16_sbase(gSA, voffSA + (unsigned)h * 16, slot);
    async_copy16_sbase(gSB, voffSB + (unsigned)h * 16, slot + BM * 16);
  };

  // ---- fragment reads: lane (l16, kg) of sub-step ks wants chunk 2 kg + ks of row l16 (+ 16 t)
  unsigned adrA[KS], adrB[KS];
  {
    const unsigned s = (l16 >> 1) & 7;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      const unsigned slot = ((2 * kg + ks) ^ s) * 16;
      adrA[ks] = lds0 + (wm * 128 + l16) * ROWB + slot;
      adrB[ks] = lds0 + A_BYTES + (wn * 128 + l16) * ROWB + slot;
    }
  }
  struct Frags { i32x4 a[MT]; i32x4 b[NT]; };
  Frags f[2];
  auto read_one = [&](auto OP_, auto P_, auto KS_, Frags& dst) {
    constexpr int op = decltype(OP_)::value, P = decltype(P_)::value, ks = decltype(KS_)::value;
    constexpr unsigned so = P * STAGE;
    if constexpr (op < MT) dst.a[op] = lds_read_b128<op * 16 * ROWB>(adrA[ks] + so);
    else dst.b[op - MT] = lds_read_b128<(op - MT) * 16 * ROWB>(adrB[ks] + so);
  };
  auto pin = [&](Frags& x) {
    static_for<MT>([&](auto T_) { lds_use(x.a[decltype(T_)::value]); });
    static_for<NT>([&](auto T_) { lds_use(x.b[decltype(T_)::value]); });
  };
  // scales of a K step: the dword holding this lane's two bytes, shifted so that they sit in bytes 0 and 1
  const unsigned adrSA = lds0 + SC_BASE + (wm * 128 + l16) * 16 + (kg >> 1) * 4;
  const unsigned adrSB = lds0 + SC_BASE + BM * 16 + (wn * 128 + l16) * 16 + (kg >> 1) * 4;
  const int sshift = 16 * (kg & 1);
  int sa[2][MT], sb[2][NT];
  auto read_scales = [&](auto SET_, auto OFF_) {   // OFF: slot * SC_SLOT + (K step & 1) * 8
    constexpr int set = decltype(SET_)::value, off = decltype(OFF_)::value;
    static_for<MT>([&](auto T_) { constexpr int t = decltype(T_)::value; sa[set][t] = lds_read_b32<off + t * 256>(adrSA); });
    static_for<NT>([&](auto T_) { constexpr int t = decltype(T_)::value; sb[set][t] = lds_read_b32<off + t * 256>(adrSB); });
  };
  auto fix_scales = [&](auto SET_) {
    constexpr int set = decltype(SET_)::value;
    static_for<MT>([&](auto T_) { constexpr int t = decltype(T_)::value; lds_use(sa[set][t]); sa[set][t] = (int)((unsigned)sa[set][t] >> sshift); });
    static_for<NT>([&](auto T_) { constexpr int t = decltype(T_)::value; lds_use(sb[set][t]); sb[set][t] = (int)((unsigned)sb[set][t] >> sshift); });
  };

  f32x4 acc[MT][NT];
  auto zero_acc = [&]() {
#pragma unroll
    for (int i = 0; i < MT; i++)
#pragma unroll
      for (int j = 0; j < NT; j++) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  };
  zero_acc();

  // ---- prologue
  using I0 = std::integral_constant<int, 0>; using I1 = std::integral_constant<int, 1>;
  using T = std::true_type; using F = std::false_type;
  issue_scales(0);
  static_for<16>([&](auto J_) { issue(J_, 0, lds0); });
  static_for<16>([&](auto J_) { issue(J_, 1, lds0 + STAGE); });
  wait_vmcnt<16>();
  block_barrier();
  static_for<NRD>([&](auto OP_) { read_one(OP_, I0{}, I0{}, f[0]); });
  read_scales(I0{}, I0{});
  lds_wait<0>();
  fix_scales(I0{});

  // K step U (0..3 within a group of four: stage U & 1, scale slot U >> 1, scale set U & 1)
  auto step = [&](auto U_, int fk) {   // fk: the K step (of the fill tile) that this step's loads fetch
    constexpr int U = decltype(U_)::value, P = U & 1, set = U & 1;
    // sub-step 0
    static_for<NM>([&](auto N_) {
      constexpr int n = decltype(N_)::value, i = n / NT, j = n % NT;
      mfma16_mxfp4<0>(f[0].b[j], f[0].a[i], acc[i][j], sb[set][j], sa[set][i]);
      if constexpr (n % 2 == 0 && n / 2 < NRD) read_one(std::integral_constant<int, n / 2>{}, std::integral_constant<int, P>{}, I1{}, f[1]);
      if constexpr (n % 2 == 1) __builtin_amdgcn_sched_barrier(0);
    });
    // sub-step 1: meet, then read the next step's first fragments and scales and refill this stage
    lds_wait<0>();
    pin(f[1]);
    wait_vmcnt<0>();
    block_barrier();
    static_for<NM>([&](auto N_) {
      constexpr int n = decltype(N_)::value, i = n / NT, j = n % NT;
      mfma16_mxfp4<1>(f[1].b[j], f[1].a[i], acc[i][j], sb[set][j], sa[set][i]);
      if constexpr (n % 2 == 0 && n / 2 < NRD) read_one(std::integral_constant<int, n / 2>{}, std::integral_constant<int, P ^ 1>{}, I0{}, f[0]);
      if constexpr (n == 32)
        read_scales(std::integral_constant<int, set ^ 1>{}, std::integral_constant<int, (((U + 1) & 3) >> 1) * SC_SLOT + ((U + 1) & 1) * 8>{});
      if constexpr (n % 4 == 1) issue(std::integral_constant<int, n / 4>{}, fk, lds0 + P * STAGE);   // one per 64 cycles
      // (the scales of the K steps fk, fk + 1 are requested in the even steps, into the slot that the pair
      // two steps back used: its last reader was the read for the previous step, issued a step ago)
      // (after the last operand load: the eight loads of an operand share the M0 value that the first one sets)
      if constexpr (P == 0 && n == 62) issue_scales(fk >> 1);
      if constexpr (n % 2 == 1) __builtin_amdgcn_sched_barrier(0);
    });
    // everything requested above has landed before the registers are touched again
    lds_wait<0>();
    pin(f[0]);
    fix_scales(std::integral_constant<int, set ^ 1>{});
  };
  using I2 = std::integral_constant<int, 2>; using I3 = std::integral_constant<int, 3>;
  lds_wait<0>();
  pin(f[0]);
  // The fill cursor runs two K steps ahead of the MFMAs, across tile boundaries; behind the last tile it
  // wraps to that tile's first steps again (fetched into stages nobody reads any more), which keeps the
  // loop, the number of loads in flight and every wait uniform.
  int fk = 2, ftile = tile;
  auto advance = [&]() {
    if (++fk == nk) {
      fk = 0;
      if (ftile + (int)gridDim.x < ntiles) {
        ftile += gridDim.x;
        int fm, fn;
        grouped_tile(xcd_remap(ftile, ntiles), num_m, num_n, p.group_m, fm, fn);
        set_fill_tile(fm, fn);
      }
    }
  };
  while (true) {
    for (int kt = 0; kt < nk; kt += 4) {
      step(I0{}, fk); advance();
      step(I1{}, fk); advance();
      step(I2{}, fk); advance();
      step(I3{}, fk); advance();
      if (kt + 4 >= nk_last) mfma_retire();
    }
    mfma_drain(acc);
    int em = pm * BM + wm * 128, en = pn * BN + wn * 128, el = l16, ek = kg;
    asm volatile("" : "+s"(em), "+s"(en), "+v"(el), "+v"(ek));   // (keeps the epilogue's address arithmetic out of the K loop)
    gemm_epilogue16<MT, NT>(acc, p, em, en, el, ek);
    tile += gridDim.x;
    if (tile >= ntiles) break;
    grouped_tile(xcd_remap(tile, ntiles), num_m, num_n, p.group_m, pm, pn);
    zero_acc();
  }
  wait_vmcnt<0>();  // nothing may still be writing LDS when the workgroup ends
#endif
}

bool gemm_wave128_mxfp4_ok(const GemmArgs& p) {
  // whole tiles, K steps in groups of four (K a multiple of 1024 elements), scale rows that a 16-byte load can fetch
  return p.M % 256 == 0 && p.N % 256 == 0 && p.k_bytes % 512 == 0 && p.k_bytes >= 512 &&
         p.lda * 8 + p.k_bytes < (1ll << 31) && p.ldb * 8 + p.k_bytes < (1ll << 31) &&
         p.lds_a % 16 == 0 && p.lds_b % 16 == 0 && ((uintptr_t)p.sA | (uintptr_t)p.sB) % 16 == 0 &&
         p.lds_a * 64 + p.k_bytes / 16 < (1ll << 31) && p.lds_b * 64 + p.k_bytes / 16 < (1ll << 31);
}

int gemm_wave128_mxfp4_launch(const GemmArgs& p, hipStream_t stream) {
  constexpr int smem = 2 * 2 * 256 * 128 + 2 * 512 * 16;
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)gemm_wave128_mxfp4_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) return (int)e;
    attr_set = true;
  }
  const int tiles = (p.M / 256) * (p.N / 256);
  const int grid = wave128_grid(tiles, p.num_programs);
  gemm_wave128_mxfp4_kernel<<<dim3(grid), dim3(256), smem, stream>>>(p);
  return (int)hipGetLastError();
}

bool gemm_wave128_ok(const GemmArgs& p, bool b_kmajor) {
  // whole tiles, an even number (>= 2) of 128-byte K steps, 32-bit lane offsets
  if (!(p.M % 256 == 0 && p.N % 256 == 0 && p.k_bytes % 256 == 0 && p.k_bytes >= 256)) return false;
  if (p.lda * 8 + p.k_bytes >= (1ll << 31)) return false;
  // (row-major B: the per-load XOR of the column group acts on the whole lane offset, so the row term
  // in it - a multiple of the pitch - must leave the bits of the 512-byte tile row alone)
  return b_kmajor ? p.ldb * 8 + p.k_bytes < (1ll << 31) : (p.ldb % 512 == 0 && (int64_t)p.K * p.ldb + 512 < (1ll << 31));
}

template <typename V8, bool B_KMAJOR, bool AUX>
static int launch_wave128(const GemmArgs& p, hipStream_t stream) {
  constexpr int smem = 2 * 2 * 256 * 128;
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)gemm_wave128_kernel<V8, B_KMAJOR, AUX>, hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) return (int)e;
    attr_set = true;
  }
  const int tiles = (p.M / 256) * (p.N / 256);
  const int grid = wave128_grid(tiles, p.num_programs);
  gemm_wave128_kernel<V8, B_KMAJOR, AUX><<<dim3(grid), dim3(256), smem, stream>>>(p);
  return (int)hipGetLastError();
}

template <typename V8>
static int launch_wave128_grouped(const GroupedArgs& ga, int nprog, hipStream_t stream) {
  constexpr int smem = 2 * 2 * 256 * 128;
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)gemm_wave128_grouped_kernel<V8>, hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) return (int)e;
    attr_set = true;
  }
  gemm_wave128_grouped_kernel<V8><<<dim3(nprog), dim3(256), smem, stream>>>(ga);
  return (int)hipGetLastError();
}

int gemm_wave128_grouped_launch(const GroupedArgs& ga, bool bf16, int nprog, hipStream_t stream) {
  return bf16 ? launch_wave128_grouped<bf16x8>(ga, nprog, stream) : launch_wave128_grouped<f16x8>(ga, nprog, stream);
}

int gemm_wave128_launch(const GemmArgs& p, bool bf16, bool b_kmajor, hipStream_t stream) {
  if (p.aux) {
    if (b_kmajor) return bf16 ? launch_wave128<bf16x8, true, true>(p, stream) : launch_wave128<f16x8, true, true>(p, stream);
    return bf16 ? launch_wave128<bf16x8, false, true>(p, stream) : launch_wave128<f16x8, false, true>(p, stream);
  }
  if (b_kmajor) return bf16 ? launch_wave128<bf16x8, true, false>(p, stream) : launch_wave128<f16x8, true, false>(p, stream);
  return bf16 ? launch_wave128<bf16x8, false, false>(p, stream) : launch_wave128<f16x8, false, false>(p, stream);
}

}  // namespace mi355

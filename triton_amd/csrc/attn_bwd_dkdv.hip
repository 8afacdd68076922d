// Flash-attention backward for gfx950, dK/dV pass (see attn_bwd.hip for the algorithm, the
// reference lines it follows and the operand plan).  A file of its own because it is compiled
// with the accumulators in AGPRs - dK and dV are touched by MFMAs only - while the kernels in
// attn_bwd.hip want theirs in architectural VGPRs.
#include "attn_tiles.h"
#include "launch.h"

namespace mi355 {

template <typename V8> struct ElemB;
template <> struct ElemB<bf16x8> { using type = __bf16; };
template <> struct ElemB<f16x8> { using type = _Float16; };

// ---------------------------------------------------------------------------------------------
// dK/dV: one wave owns 32 key rows (K / V fragments and both accumulators in registers: one wave
// per SIMD); Q / dO tiles of 64 rows stream through a ring of four LDS stages, each carrying the
// M and delta values of its rows.
//
// With a single wave per SIMD nothing hides a latency for free, so the loop is software
// pipelined over the 32-row query tiles t = 0, 1, ...:
//     A(t):  S = Q K^T and dP = dO V^T          (2 * D/16 MFMAs, row-wise LDS operands)
//     X(t):  p = exp2(S*s2 - M), ds = p (dP - delta), rounded to the input type   (VALU)
//     C(t):  dV^T += dO^T p,  dK^T += Q^T ds    (2 * D/16 MFMAs, transposed LDS operands)
// run as  ... [A(t+1) with X(t) and the transposed reads of t in between] [C(t) with the row-wise
// reads of t+2 and the M/delta reads of t+1 in between] ...  so every MFMA group covers the other
// pipes' work of its neighbours.  Tiles that lie entirely above the causal diagonal of a wave are
// multiplied like the diagonal one: the mask turns p and ds into exact zeros.
// One barrier per stage (two tiles), placed where every wave has finished reading the stage
// before and has seen its own share of the next one arrive; the stage before is refilled there,
// three stages ahead.
// ---------------------------------------------------------------------------------------------
// S and dP MFMAs issued as inline assembly so that their results land in architectural VGPRs
// while the compiler keeps the dK / dV accumulators (and, through the "a" constraint, the resident
// K / V fragments) in AGPRs: the softmax and dS arithmetic then reads them directly instead of
// through one v_accvgpr_read per value.  The compiler inserts no hazard waits for these: the
// kernel's schedule provides them - a set of S / dP tiles is consumed one phase (at least sixteen
// MFMAs) after the last MFMA that writes it, and the operands come from LDS reads and global
// loads (waited for by count), never from VALU results.
// SETTLE: the padded form does feed VALU results in - its K / V fragments are zero-filled, live in VGPRs and are
// copied into AGPRs (v_accvgpr_write) right in front of the statement; an MFMA must not read a register within
// two issue slots of a VALU write (the compiler keeps that distance for the MFMAs it knows), so the statement
// starts with two idle slots.  tests/test_isa_hazards.py checks the rule on the generated code of every kernel.
template <bool SETTLE>
__device__ __forceinline__ void mfma32_first_v(f32x16& d, bf16x8 a, bf16x8 b) {
#if MI355_DEVICE_PASS
  if constexpr (SETTLE) asm volatile("s_nop 1\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(d) : "v"(a), "a"(b));
  else asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(d) : "v"(a), "a"(b));
#endif
}
template <bool SETTLE>
__device__ __forceinline__ void mfma32_first_v(f32x16& d, f16x8 a, f16x8 b) {
#if MI355_DEVICE_PASS
  if constexpr (SETTLE) asm volatile("s_nop 1\n\tv_mfma_f32_32x32x16_f16 %0, %1, %2, 0" : "=&v"(d) : "v"(a), "a"(b));
  else asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, 0" : "=&v"(d) : "v"(a), "a"(b));
#endif
}
template <bool SETTLE>
__device__ __forceinline__ void mfma32_acc_v(f32x16& d, bf16x8 a, bf16x8 b) {
#if MI355_DEVICE_PASS
  if constexpr (SETTLE) asm volatile("s_nop 1\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(d) : "v"(a), "a"(b));
  else asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(d) : "v"(a), "a"(b));
#endif
}
template <bool SETTLE>
__device__ __forceinline__ void mfma32_acc_v(f32x16& d, f16x8 a, f16x8 b) {
#if MI355_DEVICE_PASS
  if constexpr (SETTLE) asm volatile("s_nop 1\n\tv_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(d) : "v"(a), "a"(b));
  else asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(d) : "v"(a), "a"(b));
#endif
}

// PAD (D = 64 only): p.d_real = 16 or 32 columns exist in memory (see attn_bwd_dq_kernel).
template <typename V8, int D, int NW, bool PAD = false>
__global__ __launch_bounds__(NW * 64, 1) void attn_bwd_dkdv_kernel(AttnArgs p) {
  using S = typename ElemB<V8>::type;
  typedef __attribute__((ext_vector_type(4))) S S4;
  constexpr int BN = NW * 32, BM = 64, RB = D * 2, KSQ = D / 16, DT = D / 32, NS = 4;
  using Tile = AttnTile<RB, BM, NW>;
  constexpr int TILE = Tile::BYTES;
  constexpr int STAGE = 2 * TILE + 2 * BM * 4;  // Q tile | dO tile | M rows | delta rows
  constexpr int kShare = 2 * Tile::INST + 1;    // direct loads per wave and stage

  extern __shared__ __attribute__((aligned(1024))) char smem[];
  LDS_PTR(char) const lds = (LDS_PTR(char))smem;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // scalar: branches on it are uniform
  const int l32 = lane & 31, g = lane >> 5, i16 = lane & 15, q4 = lane >> 4;

  const int nkb = (p.N + BN - 1) / BN;
  int pid = xcd_remap(blockIdx.x, nkb * p.Z * p.H);
  const int hz = pid / nkb;
  const int kbk = pid % nkb;  // causal: low key blocks have the most work, ascending order = longest first
  const int z = hz / p.H, h = hz % p.H;
  const int n0 = kbk * BN, nrow0 = n0 + wave * 32;

  const int64_t head_off = ((int64_t)z * p.sq[0] + (int64_t)h * p.sq[1]) * 2;
  const int64_t pitch = p.sq[2] * 2;
  const char* qbase = p.q + head_off;
  const char* dobase = p.d_o + head_off;
  const float* lse = p.lse + (int64_t)hz * p.N;
  const float* delta = p.delta + (int64_t)hz * p.N;

  // K / V fragments of this wave's key rows: lane (row l32, half g) holds X[row][16*ks + 8*g .. +8]
  V8 kf[KSQ], vf[KSQ];
  {
    int r = min(nrow0 + l32, p.N - 1);
    const char* sk = p.k + head_off + (int64_t)r * pitch + g * 16;
    const char* sv = p.v + head_off + (int64_t)r * pitch + g * 16;
#pragma unroll
    for (int ks = 0; ks < KSQ; ks++) {
      if (!PAD || ks * 32 + g * 16 < p.d_real * 2) {
        kf[ks] = *(const V8*)(sk + ks * 32);
        vf[ks] = *(const V8*)(sv + ks * 32);
      } else {
        kf[ks] = V8{};
        vf[ks] = V8{};
      }
    }
  }

  // query rows m >= n0 (causal) or all of them, in stages of BM rows
  const int m_begin = p.causal ? (n0 / BM) * BM : 0;
  const int nsteps = (p.N - m_begin + BM - 1) / BM;
  const int ncol = nrow0 + l32;  // this lane's key row

  // direct loads: scalar tile base + 32-bit lane offset (the host bounds the row pitch)
  unsigned offQD[Tile::INST];
  bool present[Tile::INST];
#pragma unroll
  for (int i = 0; i < Tile::INST; i++) {
    offQD[i] = (unsigned)Tile::off(pitch, wave, lane, i);
    present[i] = !PAD || Tile::chunk_present(wave, lane, i, p.d_real * 2);
  }
  if constexpr (PAD) {
    lds_zero(lds, NS * STAGE, tid, NW * 64);
    __syncthreads();
  }
  const char* const qsrc0 = qbase + (int64_t)m_begin * pitch;
  const char* const dsrc0 = dobase + (int64_t)m_begin * pitch;
  const unsigned lds_base = lds_addr(lds);
  // even waves copy the stage's 64 M values, odd waves its 64 deltas (4 bytes per lane; the
  // duplicates keep the number of loads per wave uniform for the partial waits)
  const float* src_stat = ((wave & 1) == 0 ? lse : delta) + m_begin + lane;
  // stage-step js (clamped to the last one) into ring slot js % NS: nine loads per wave (kShare), issued as a burst
  // in the prologue and one at a time between the MFMAs of the loop (a burst there held the wave up for about 380
  // cycles per stage: with one wave per SIMD nothing else issues while the memory pipeline takes the loads)
  struct StageSrc { const char* q; const char* d; const float* stat; unsigned lds; };
  auto stage_src = [&](int js) {
    const int jc = min(js, nsteps - 1);
    const int64_t off = (int64_t)jc * BM * pitch;
    return StageSrc{qsrc0 + off, dsrc0 + off, src_stat + jc * BM, lds_base + (js % NS) * STAGE};
  };
  auto stage_load = [&](auto I_, const StageSrc& ss) {   // load number I of kShare
    constexpr int I = decltype(I_)::value;
    if constexpr (I < 2 * Tile::INST) {
      constexpr int i = I >> 1;
      // (every row has chunks that are present, so every wave still issues every load: the counts of the partial
      // waits below stay what they are)
      if (present[i]) {
        if constexpr ((I & 1) == 0) async_copy16_sbase(ss.q, offQD[i], ss.lds + (i * NW + wave) * 1024);
        else async_copy16_sbase(ss.d, offQD[i], ss.lds + TILE + (i * NW + wave) * 1024);
      }
    } else {
      async_copy4_asm(ss.stat, ss.lds + 2 * TILE + (wave & 1) * (BM * 4));
    }
  };
  auto issue_stage = [&](int js) {
    const StageSrc ss = stage_src(js);
    static_for<kShare>([&](auto I_) { stage_load(I_, ss); });
  };

  // per-lane LDS offsets inside a stage: row-wise operand per k-step, transposed operand per
  // (column block, half); stage, tile and sub-row offsets are added as scalars / immediates
  const RowRead<RB> rr(l32, g);
  const TrRead<RB> tt(i16, q4);
  unsigned ra[KSQ], ta[DT][2];
#pragma unroll
  for (int ks = 0; ks < KSQ; ks++) ra[ks] = rr.rowb + (rr.xk ^ (ks * 32));
#pragma unroll
  for (int c = 0; c < DT; c++)
#pragma unroll
    for (int h2 = 0; h2 < 2; h2++) ta[c][h2] = tt.tl ^ ((c << 6) | (h2 << 5));
  const unsigned lds0 = lds_addr(lds);

  f32x16 dk[DT], dv[DT];
#pragma unroll
  for (int c = 0; c < DT; c++)
#pragma unroll
    for (int r = 0; r < 16; r++) { dk[c][r] = 0.f; dv[c][r] = 0.f; }
  f32x16 sacc[2], dpacc[2];   // S and dP of the tile being multiplied / the tile being exponentiated
  i32x4 rq[KSQ], rd[KSQ];     // row-wise Q / dO operands of the next A
  i32x2 tq[2][DT][2], td[2][DT][2];  // transposed Q / dO operands of the next C
  i32x4 mvi[4], dli[4];       // M and delta of the 16 query rows this lane's S registers stand for
  V8 pf[2], dsf[2];           // p and ds as B operands of C, per 16-row k-step

  const float qk_scale = p.sm_scale * 1.4426950408889634f;

  // ---- pieces of the pipeline; MT = which 32-row half of the stage the tile is
  auto read_rows = [&](auto I_, auto MT_, unsigned sbase) {  // read number I of 2*KSQ
    constexpr int i = decltype(I_)::value, mt = decltype(MT_)::value, ks = i >> 1;
    if constexpr ((i & 1) == 0) rq[ks] = lds_read_b128<mt * 32 * RB>(sbase + ra[ks]);
    else rd[ks] = lds_read_b128<TILE + mt * 32 * RB>(sbase + ra[ks]);
  };
  auto read_stats = [&](auto I_, auto MT_, unsigned sbase) {  // read number I of 8
    constexpr int i = decltype(I_)::value, mt = decltype(MT_)::value, rg = i >> 1;
    if constexpr ((i & 1) == 0) mvi[rg] = lds_read_b128<2 * TILE + mt * 128 + rg * 32>(sbase + g * 16);
    else dli[rg] = lds_read_b128<2 * TILE + BM * 4 + mt * 128 + rg * 32>(sbase + g * 16);
  };
  auto read_tr = [&](auto I_, auto MT_, unsigned sbase) {  // read number I of 8*DT
    constexpr int i = decltype(I_)::value, mt = decltype(MT_)::value;
    constexpr int which = i & 1, h2 = (i >> 1) & 1, c = (i >> 2) % DT, t = i / (4 * DT);
    constexpr int imm = (mt * 32 + 16 * t + 8 * h2) * RB;
    if constexpr (which == 0) tq[t][c][h2] = lds_read_tr16_b64<imm>(sbase + ta[c][h2]);
    else td[t][c][h2] = lds_read_tr16_b64<TILE + imm>(sbase + ta[c][h2]);
  };
  auto settle_rows = [&]() {
    lds_wait<0>();
#pragma unroll
    for (int ks = 0; ks < KSQ; ks++) { lds_use(rq[ks]); lds_use(rd[ks]); }
  };
  auto settle_stats = [&]() {
#pragma unroll
    for (int rg = 0; rg < 4; rg++) { lds_use(mvi[rg]); lds_use(dli[rg]); }
  };
  auto settle_tr = [&]() {
    lds_wait<0>();
#pragma unroll
    for (int t = 0; t < 2; t++)
#pragma unroll
      for (int c = 0; c < DT; c++)
#pragma unroll
        for (int h2 = 0; h2 < 2; h2++) { lds_use(tq[t][c][h2]); lds_use(td[t][c][h2]); }
  };
  // X: elements r0 .. r0+n-1 of the tile whose S / dP sit in set PAR; mrow0 = its first query row
  auto softmax_part = [&](auto PAR_, auto R0_, auto N_, int mrow0, auto MASKED_) {
    constexpr int par = decltype(PAR_)::value, r0 = decltype(R0_)::value, n = decltype(N_)::value;
    constexpr bool masked = decltype(MASKED_)::value;
#pragma unroll
    for (int r = r0; r < r0 + n; r++) {
      const float mval = __builtin_bit_cast(f32x4, mvi[r >> 2])[r & 3];
      const float dval = __builtin_bit_cast(f32x4, dli[r >> 2])[r & 3];
      float pv = fast_exp2(fmaf(sacc[par][r], qk_scale, -mval));
      if constexpr (masked) {
        int m = mrow0 + (r >> 2) * 8 + g * 4 + (r & 3);
        if (m < ncol) pv = 0.f;
      }
      float dsv = pv * (dpacc[par][r] - dval);
      pf[r >> 3][r & 7] = (S)pv;
      dsf[r >> 3][r & 7] = (S)dsv;
    }
  };
  // A(next tile) into set PAR with X(previous tile, set PAR^1) and its transposed reads in between
  // (Every MFMA is followed by its share of the other work.  Two MFMAs back to back leave the first one's 32 cycles
  // empty: the second cannot issue before the pipe is free, and nothing behind it can issue before it - measured on
  // the kernel's own cycle counter, phase A took 977 cycles per tile = 532 of MFMAs + 285 of softmax + 204 of
  // transposed reads, every part in full.)
  auto phase_a_impl = [&](auto PAR_, auto MTX_, auto DOX_, auto MASKED_, int mrow0_x, unsigned sbase_x) {
    constexpr int par = decltype(PAR_)::value;
    constexpr bool do_x = decltype(DOX_)::value;
    constexpr int EPK = 16 / KSQ, EH = EPK / 2;                   // X elements per k-step, per MFMA
    constexpr int TRK = (8 * DT + KSQ - 2) / (KSQ - 1), TH = (TRK + 1) / 2;   // transposed reads per k-step (none in the last), first share
    settle_rows();
    settle_stats();
    static_for<KSQ>([&](auto KS_) {
      constexpr int ks = decltype(KS_)::value;
      if constexpr (ks == 0) mfma32_first_v<PAD>(sacc[par], __builtin_bit_cast(V8, rq[0]), kf[0]);
      else mfma32_acc_v<PAD>(sacc[par], __builtin_bit_cast(V8, rq[ks]), kf[ks]);
      if constexpr (do_x) {
        static_for<TH>([&](auto O_) {
          constexpr int i = ks * TRK + decltype(O_)::value;
          if constexpr (i < 8 * DT) read_tr(std::integral_constant<int, i>{}, MTX_, sbase_x);
        });
        softmax_part(std::integral_constant<int, par ^ 1>{}, std::integral_constant<int, ks * EPK>{},
                     std::integral_constant<int, EH>{}, mrow0_x, MASKED_);
      }
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (ks == 0) mfma32_first_v<PAD>(dpacc[par], __builtin_bit_cast(V8, rd[0]), vf[0]);
      else mfma32_acc_v<PAD>(dpacc[par], __builtin_bit_cast(V8, rd[ks]), vf[ks]);
      if constexpr (do_x) {
        static_for<TRK - TH>([&](auto O_) {
          constexpr int i = ks * TRK + TH + decltype(O_)::value;
          if constexpr (i < 8 * DT) read_tr(std::integral_constant<int, i>{}, MTX_, sbase_x);
        });
        softmax_part(std::integral_constant<int, par ^ 1>{}, std::integral_constant<int, ks * EPK + EH>{},
                     std::integral_constant<int, EPK - EH>{}, mrow0_x, MASKED_);
      }
      __builtin_amdgcn_sched_barrier(0);
    });
  };

  // C(tile) with the row-wise reads of the tile after next (stage sbase_r, half MTR) and the
  // M / delta reads of the next tile (stage sbase_s, half MTS) in between
  // LOADS: this phase also requests the next stage of the ring, one load behind each MFMA pair's first MFMA
  auto phase_c = [&](auto MTR_, unsigned sbase_r, auto MTS_, unsigned sbase_s, auto LOADS_, const StageSrc& ss) {
    constexpr int NM = 2 * DT;               // MFMA pairs
    constexpr int NRD = 2 * KSQ + 8;         // reads to place
    constexpr int PER = (NRD + NM - 3) / (NM - 2), PH = (PER + 1) / 2;   // per pair (none in the last two), first share
    constexpr bool loads = decltype(LOADS_)::value;
    constexpr int LPP = (kShare + NM - 1) / NM;   // loads per pair
    auto reads = [&](auto FROM_, auto N_) {
      static_for<decltype(N_)::value>([&](auto O_) {
        constexpr int i = decltype(FROM_)::value + decltype(O_)::value;
        if constexpr (i < 2 * KSQ) read_rows(std::integral_constant<int, i>{}, MTR_, sbase_r);
        else if constexpr (i < NRD) read_stats(std::integral_constant<int, i - 2 * KSQ>{}, MTS_, sbase_s);
      });
    };
    settle_tr();
    static_for<NM>([&](auto N_) {
      constexpr int n = decltype(N_)::value, t = n / DT, c = n % DT;
      i32x4 qt = __builtin_shufflevector(tq[t][c][0], tq[t][c][1], 0, 1, 2, 3);
      i32x4 dt = __builtin_shufflevector(td[t][c][0], td[t][c][1], 0, 1, 2, 3);
      dv[c] = mfma32(__builtin_bit_cast(V8, dt), pf[t], dv[c]);
      reads(std::integral_constant<int, n * PER>{}, std::integral_constant<int, PH>{});
      if constexpr (loads) {
        static_for<LPP>([&](auto L_) {
          constexpr int l = n * LPP + decltype(L_)::value;
          if constexpr (l < kShare) stage_load(std::integral_constant<int, l>{}, ss);
        });
      }
      __builtin_amdgcn_sched_barrier(0);
      dk[c] = mfma32(__builtin_bit_cast(V8, qt), dsf[t], dk[c]);
      reads(std::integral_constant<int, n * PER + PH>{}, std::integral_constant<int, PER - PH>{});
      __builtin_amdgcn_sched_barrier(0);
    });
  };
  using I0 = std::integral_constant<int, 0>;
  using I1 = std::integral_constant<int, 1>;

  // ---- prologue: three stages in flight; A(0) alone; operands of A(1) and M/delta of tile 0
#pragma unroll
  for (int js = 0; js < NS - 1; js++) issue_stage(js);
  wait_vmcnt<(NS - 2) * kShare>();
  __builtin_amdgcn_sched_barrier(0);
  block_barrier();
  __builtin_amdgcn_sched_barrier(0);
  static_for<2 * KSQ>([&](auto I_) { read_rows(I_, I0{}, lds0); });
  static_for<8>([&](auto I_) { read_stats(I_, I0{}, lds0); });
  phase_a_impl(I0{}, I0{}, std::false_type{}, std::false_type{}, 0, 0u);
  static_for<2 * KSQ>([&](auto I_) { read_rows(I_, I1{}, lds0); });

  // one stage (two tiles) of the pipeline
  auto stage_step = [&](int j, auto MASKED_) {
    const unsigned sb_cur = lds0 + (j % NS) * STAGE;
    const unsigned sb_nxt = lds0 + ((j + 1) % NS) * STAGE;
    const int ms = m_begin + j * BM;
    // A(2j+1) | X(2j), transposed reads of tile 2j
    phase_a_impl(I1{}, I0{}, std::true_type{}, MASKED_, ms, sb_cur);
    // every wave is done with stage j-1 and has seen its share of stage j+1 arrive
    wait_vmcnt<kShare>();
    __builtin_amdgcn_sched_barrier(0);
    block_barrier();
    __builtin_amdgcn_sched_barrier(0);
    const StageSrc ss = stage_src(j + NS - 1);
    // C(2j) | row-wise reads of tile 2j+2 (next stage), M/delta of tile 2j+1, the loads of stage j + NS - 1
    phase_c(I0{}, sb_nxt, I1{}, sb_cur, std::true_type{}, ss);
    // A(2j+2) | X(2j+1), transposed reads of tile 2j+1
    phase_a_impl(I0{}, I1{}, std::true_type{}, MASKED_, ms + 32, sb_cur);
    // C(2j+1) | row-wise reads of tile 2j+3, M/delta of tile 2j+2
    phase_c(I1{}, sb_nxt, I0{}, sb_nxt, std::false_type{}, ss);
  };
  // causal: the workgroup's 128 key rows meet the diagonal in its first two stages (query rows
  // n0 .. n0+127); only those pay for the mask
  const int nmasked = p.causal ? min(2, nsteps) : 0;
  for (int j = 0; j < nmasked; j++) stage_step(j, std::true_type{});
  for (int j = nmasked; j < nsteps; j++) stage_step(j, std::false_type{});
  // nothing may still be writing this workgroup's LDS when it retires - nor this wave's registers: the last C phase
  // has read the rows and the M / delta values of tiles that do not follow, and the compiler, which takes those
  // registers as written when the read was issued, would otherwise put dK / dV values into them ahead of the wait
  // (a late read then lands on top of a result)
  wait_all();
  settle_rows();
  settle_stats();

  // dK and dV rows through LDS (store_rows_transposed), one after the other through the same 32 x D elements per
  // wave at the start of the ring - once every wave has left the loop
  __syncthreads();
  if (nrow0 < p.N) {
    const unsigned mine = lds0 + wave * 32 * RB;
    store_rows_transposed<S, D, PAD>(dk, p.sm_scale, mine, p.dk + head_off + (int64_t)nrow0 * pitch, pitch, p.N - nrow0, p.d_real, lane);
    store_rows_transposed<S, D, PAD>(dv, 1.f, mine, p.dv + head_off + (int64_t)nrow0 * pitch, pitch, p.N - nrow0, p.d_real, lane);
  }
}


// ---------------------------------------------------------------------------------------------
// dK/dV for head_dim 256.  K, V fragments (128 registers) plus both accumulators (256 more at this
// width) do not fit one wave, so a workgroup owns 128 key rows and HALF of the output columns:
// program 2 i + h computes dK[:, 128 h .. 128 h + 127] and dV[:, same] of key block i.  S and dP
// need the whole head dimension and are computed by both programs (6 products' worth of MFMAs
// for the 4 that count per output half - the price of keeping every accumulator in registers
// and of needing no workspace and no atomics).  Plain structure, two LDS stages of a Q and a dO
// tile (64 rows x 512 bytes each), one barrier per stage: this width is about coverage of the
// reference surface (python/tutorials/06-fused-attention.py:447 admits HEAD_DIM 256), not speed.
// ---------------------------------------------------------------------------------------------
template <typename V8, int D, int NW>
__global__ __launch_bounds__(NW * 64, 1) void attn_bwd_dkdv_split_kernel(AttnArgs p) {
  using S = typename ElemB<V8>::type;
  typedef __attribute__((ext_vector_type(4))) S S4;
  constexpr int BN = NW * 32, BM = 64, RB = D * 2, KSQ = D / 16, DH = D / 2, DT = DH / 32;
  using Tile = AttnTile<RB, BM, NW>;
  constexpr int TILE = Tile::BYTES;

  extern __shared__ __attribute__((aligned(1024))) char smem[];
  LDS_PTR(char) const lds = (LDS_PTR(char))smem;  // [stage][Q tile | dO tile]

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, g = lane >> 5, i16 = lane & 15, q4 = lane >> 4;

  const int nkb = (p.N + BN - 1) / BN;
  const int dhalf = blockIdx.x & 1;
  const int pid = blockIdx.x >> 1;
  const int hz = pid / nkb, kbk = pid % nkb;
  const int z = hz / p.H, h = hz % p.H;
  const int n0 = kbk * BN, nrow0 = n0 + wave * 32;
  const int ncol = nrow0 + l32;   // this lane's key row

  const int64_t head_off = ((int64_t)z * p.sq[0] + (int64_t)h * p.sq[1]) * 2;
  const int64_t pitch = p.sq[2] * 2;
  const char* qbase = p.q + head_off;
  const char* dobase = p.d_o + head_off;
  const float* lse = p.lse + (int64_t)hz * p.N;
  const float* delta = p.delta + (int64_t)hz * p.N;

  V8 kf[KSQ], vf[KSQ];
  {
    const int r = min(ncol, p.N - 1);
    const char* sk = p.k + head_off + (int64_t)r * pitch + g * 16;
    const char* sv = p.v + head_off + (int64_t)r * pitch + g * 16;
#pragma unroll
    for (int ks = 0; ks < KSQ; ks++) {
      kf[ks] = *(const V8*)(sk + ks * 32);
      vf[ks] = *(const V8*)(sv + ks * 32);
    }
  }

  const int m_begin = p.causal ? (n0 / BM) * BM : 0;
  const int nsteps = (p.N - m_begin + BM - 1) / BM;

  unsigned offQD[Tile::INST];
#pragma unroll
  for (int i = 0; i < Tile::INST; i++) offQD[i] = (unsigned)Tile::off(pitch, wave, lane, i);
  const unsigned lds_base = lds_addr(lds);
  auto issue = [&](int j, int stage) {
    const unsigned qd = lds_base + stage * (2 * TILE), dd = qd + TILE;
    const char* qsrc = qbase + (int64_t)(m_begin + j * BM) * pitch;
    const char* dsrc = dobase + (int64_t)(m_begin + j * BM) * pitch;
#pragma unroll
    for (int i = 0; i < Tile::INST; i++) {
      async_copy16_sbase(qsrc, offQD[i], qd + (i * NW + wave) * 1024);
      async_copy16_sbase(dsrc, offQD[i], dd + (i * NW + wave) * 1024);
    }
  };

  const RowRead<RB> rr(l32, g);
  TrRead<RB> tt(i16, q4);
  tt.tl ^= (unsigned)dhalf << 8;   // column blocks 4 h .. 4 h + 3: 256 bytes further, and the swizzle XOR leaves bit 8 alone

  f32x16 dk[DT], dv[DT];
#pragma unroll
  for (int c = 0; c < DT; c++)
#pragma unroll
    for (int r = 0; r < 16; r++) { dk[c][r] = 0.f; dv[c][r] = 0.f; }

  const float qk_scale = p.sm_scale * 1.4426950408889634f;

  issue(0, 0);
  wait_all();
  __syncthreads();

  for (int j = 0; j < nsteps; j++) {
    const int stage = j & 1;
    if (j + 1 < nsteps) issue(j + 1, stage ^ 1);
    const unsigned qb = lds_base + stage * (2 * TILE), db = qb + TILE;
    const int ms = m_begin + j * BM;
    static_for<2>([&](auto A_) {
      constexpr int a = decltype(A_)::value;
      const int mt0 = ms + a * 32;   // first query row of this 32-row tile
      // under the causal mask a tile whose rows all lie above this wave's key rows contributes nothing
      if (!p.causal || mt0 + 31 >= nrow0) {
        f32x16 s, dp;
#pragma unroll
        for (int r = 0; r < 16; r++) { s[r] = 0.f; dp[r] = 0.f; }
        i32x4 qf[2], df[2];
        qf[0] = lds_read_b128<a * 32 * RB>(rr.template addr<0>(qb));
        df[0] = lds_read_b128<a * 32 * RB>(rr.template addr<0>(db));
        static_for<KSQ>([&](auto KS_) {
          constexpr int ks = decltype(KS_)::value;
          constexpr int cur = ks & 1, nxt = cur ^ 1;
          if constexpr (ks + 1 < KSQ) {
            qf[nxt] = lds_read_b128<a * 32 * RB>(rr.template addr<ks + 1>(qb));
            df[nxt] = lds_read_b128<a * 32 * RB>(rr.template addr<ks + 1>(db));
            lds_wait<2>();
          } else {
            lds_wait<0>();
          }
          lds_use(qf[cur]);
          lds_use(df[cur]);
          s = mfma32(__builtin_bit_cast(V8, qf[cur]), kf[ks], s);      // S[q][key] = Q K^T
          dp = mfma32(__builtin_bit_cast(V8, df[cur]), vf[ks], dp);    // dP[q][key] = dO V^T
        });
        V8 pf[2], dsf[2];
        const bool masked = p.causal && mt0 < nrow0 + 32;
#pragma unroll
        for (int rg = 0; rg < 4; rg++) {
          const int mrow = min(mt0 + rg * 8 + g * 4, p.N - 4);
          const f32x4 mv = *(const f32x4*)(lse + mrow);
          const f32x4 dl = *(const f32x4*)(delta + mrow);
#pragma unroll
          for (int e = 0; e < 4; e++) {
            const int r = rg * 4 + e;
            float pv = fast_exp2(fmaf(s[r], qk_scale, -mv[e]));
            if (masked && mt0 + rg * 8 + g * 4 + e < ncol) pv = 0.f;
            const float dsv = pv * (dp[r] - dl[e]);
            pf[r >> 3][r & 7] = (S)pv;
            dsf[r >> 3][r & 7] = (S)dsv;
          }
        }
        // dV^T += dO^T p and dK^T += Q^T ds over the two k-steps of 16 query rows
        static_for<2>([&](auto T_) {
          constexpr int t = decltype(T_)::value;
          static_for<DT>([&](auto C_) {
            constexpr int c = decltype(C_)::value;
            constexpr int imm0 = (a * 32 + 16 * t) * RB, imm1 = (a * 32 + 16 * t + 8) * RB;
            i32x2 q0 = lds_read_tr16_b64<imm0>(tt.template addr<c, 0>(qb));
            i32x2 q1 = lds_read_tr16_b64<imm1>(tt.template addr<c, 1>(qb));
            i32x2 d0 = lds_read_tr16_b64<imm0>(tt.template addr<c, 0>(db));
            i32x2 d1 = lds_read_tr16_b64<imm1>(tt.template addr<c, 1>(db));
            lds_wait<0>();
            lds_use(q0); lds_use(q1); lds_use(d0); lds_use(d1);
            const i32x4 qt = __builtin_shufflevector(q0, q1, 0, 1, 2, 3);
            const i32x4 dt = __builtin_shufflevector(d0, d1, 0, 1, 2, 3);
            dv[c] = mfma32(__builtin_bit_cast(V8, dt), pf[t], dv[c]);
            dk[c] = mfma32(__builtin_bit_cast(V8, qt), dsf[t], dk[c]);
          });
        });
      }
    });
    wait_all();
    __syncthreads();
  }

  // this program's DH columns of the dK and dV rows, through LDS (the loop ended with a full wait and a barrier)
  if (nrow0 < p.N) {
    const unsigned mine = lds_addr(lds) + wave * 32 * (DH * 2);
    const int64_t at = head_off + (int64_t)nrow0 * pitch + dhalf * DH * 2;
    store_rows_transposed<S, DH, false>(dk, p.sm_scale, mine, p.dk + at, pitch, p.N - nrow0, DH, lane);
    store_rows_transposed<S, DH, false>(dv, 1.f, mine, p.dv + at, pitch, p.N - nrow0, DH, lane);
  }
}

template <typename V8>
static int launch_dkdv_256(const AttnArgs& p, hipStream_t stream) {
  constexpr int NW = 4, BN = NW * 32, D = 256;
  constexpr int smem = 2 * 2 * 64 * D * 2;
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)attn_bwd_dkdv_split_kernel<V8, D, NW>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) return (int)e;
    attr_set = true;
  }
  const int nkb = (p.N + BN - 1) / BN;
  attn_bwd_dkdv_split_kernel<V8, D, NW><<<dim3(2 * nkb * p.Z * p.H), dim3(NW * 64), smem, stream>>>(p);
  return (int)hipGetLastError();
}

template <typename V8, int D, bool PAD = false>
static int launch_dkdv(const AttnArgs& p, hipStream_t stream) {
  constexpr int NW = 4, BN = NW * 32;
  constexpr int smem = 4 * (2 * 64 * D * 2 + 2 * 64 * 4);
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)attn_bwd_dkdv_kernel<V8, D, NW, PAD>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) return (int)e;
    attr_set = true;
  }
  int nkb = (p.N + BN - 1) / BN;
  attn_bwd_dkdv_kernel<V8, D, NW, PAD><<<dim3(nkb * p.Z * p.H), dim3(NW * 64), smem, stream>>>(p);
  return (int)hipGetLastError();
}

int attn_bwd_dkdv_launch(const AttnArgs& p, bool bf16, hipStream_t stream) {
  if (p.d_real < p.D) return bf16 ? launch_dkdv<bf16x8, 64, true>(p, stream) : launch_dkdv<f16x8, 64, true>(p, stream);
  if (p.D == 256) return bf16 ? launch_dkdv_256<bf16x8>(p, stream) : launch_dkdv_256<f16x8>(p, stream);
  if (bf16) return p.D == 128 ? launch_dkdv<bf16x8, 128>(p, stream) : launch_dkdv<bf16x8, 64>(p, stream);
  return p.D == 128 ? launch_dkdv<f16x8, 128>(p, stream) : launch_dkdv<f16x8, 64>(p, stream);
}

}  // namespace mi355

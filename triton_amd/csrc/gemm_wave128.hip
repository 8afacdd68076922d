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
#include "gemm_wave128.h"

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

// The tiles `tile`, `tile + tile_step`, ... (< `tile_stop`, by default M/256 * N/256) of one problem, computed by the calling workgroup
// with the 128 KiB of LDS at `lds0`.  XCD: pass the tile numbers through the per-XCD remap first.  EPI: 0 = scales,
// activation, any output type; 1 = C has the type of the operands, no scales, no activation; 2 = 0 plus the addend;
// 3 = the lean epilogue (gemm_epilogue16_lean) with C in the operands' type.
// TAIL: K bytes need not be a multiple of 256; what is left behind the last pair of K steps (16 .. 240 bytes of
// every operand row) is multiplied after the K loop, 64 bytes at a time, through a 32 KiB LDS buffer of its own
// behind the two stages (which by then hold the next tile's first steps): plain loads with a zero fill, one
// un-pipelined sub-step each - a per-tile cost of a few microseconds that only products with such a K pay
// (the reference's own uneven-K shape 8192 x 8192 x 8176, python/test/regression/test_performance.py:46).
template <typename V8, bool B_KMAJOR, bool XCD, int EPI = 0, bool TAIL = false, int BM = 256>
__device__ __forceinline__ void gemm_wave128_tiles(const GemmArgs& p, int tile, const int tile_step, const unsigned lds0, const int tile_stop = -1) {
#if MI355_DEVICE_PASS
  // BM = 192: tiles of 192 x 256 (96 x 128 per wave) for problems whose 256 x 256 tiles would leave a quarter or more of
  // the CUs idle - only the A side changes: six direct loads per wave and K step instead of eight, six fragments
  static_assert((BM == 256 || BM == 192 || BM == 128) && !(TAIL && BM != 256), "tile heights");
  constexpr int BN = 256, ROWB = 128;
  constexpr int A_BYTES = BM * ROWB, STAGE = A_BYTES + BN * ROWB;  // 64 KiB (56 KiB)
  constexpr int MT = BM / 32, NT = 8, KS = 2;                       // 16x16 tiles per wave, 16x16x32 sub-steps per stage
  constexpr int LA = BM / 32, NLOADS = LA + 8;                      // direct loads per wave and K step: A, then B
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
  const int nk = TAIL ? (p.k_bytes / (2 * ROWB)) * 2 : p.k_bytes / ROWB;   // K steps of the pipelined loop (an even number)
  int nk_last = nk;   // the same number, but opaque: see mfma_retire
  asm volatile("" : "+s"(nk_last));

  // ---- direct loads: instruction q = 8 * wave + j moves rows 8 q .. 8 q + 7 of a tile; the swizzle of
  // those rows is 4 (q & 1) + lane / 16.  Each of a wave's loads has a lane offset of its own - row, chunk, and the
  // instruction offset taken back out - and the loads of one operand share one scalar base, the K step being
  // fetched: two scalar additions per K step are all the address arithmetic of the loop.  (Sixteen scalar
  // bases instead - one per load, rebuilt from the tile base at every load once that base changes inside the
  // loop - were 56 scalar instructions per K step.)
  const unsigned drow = lane >> 3, dslot = lane & 7;
  auto ioff_of = [](int q) constexpr { return (q - 4) * 1024; };
  unsigned voffA[LA], voffB[8];
#pragma unroll
  for (int q = 0; q < LA; q++) {
    const unsigned chunk = dslot ^ (((q & 1) * 4 + (lane >> 4)) & 7);
    voffA[q] = (drow + 8 * q) * (unsigned)p.lda + chunk * 16 - (unsigned)ioff_of(q);
  }
  // Row-major B[K, N]: the stage holds 64 k rows of 512 bytes; instruction q = 8 * wave + j moves the k rows
  // 2 q, 2 q + 1 (lane i: row i / 32, physical 16-byte chunk i % 32).  Element (k, n) lives in the 32-byte
  // column group (n / 16) ^ 2 (k & 3) ^ ((k >> 3) & 1) of its row: a transpose read is served two 16-lane
  // groups at a time - four consecutive k rows each, eight rows apart, the same 16 columns - and this
  // spreads those 8 x 32 bytes over all banks.  With k = 16 wave + 2 j + i / 32 the XOR terms are
  // 4 (j & 1) + 2 (i / 32) and (j >> 2) & 1 (which needs a pitch that is a multiple of 512 bytes).
#pragma unroll
  for (int q = 0; q < 8; q++) {
    if constexpr (B_KMAJOR) {
      const unsigned chunk = dslot ^ (((q & 1) * 4 + (lane >> 4)) & 7);
      voffB[q] = (drow + 8 * q) * (unsigned)p.ldb + chunk * 16 - (unsigned)ioff_of(q);
    } else {
      const unsigned pg = (lane & 31) >> 1, half = lane & 1;
      const unsigned v0 = (lane >> 5) * (unsigned)p.ldb + ((pg ^ (2 * (lane >> 5))) * 32) + half * 16;
      voffB[q] = (v0 ^ ((4 * (q & 1) + ((q >> 2) & 1)) * 32)) + 2 * q * (unsigned)p.ldb - (unsigned)ioff_of(q);
    }
  }
  // scalar bases of the K step the loads are fetching (two K steps ahead of the MFMAs)
  const char* fA;
  const char* fB;
  // (wave-uniform values, but the grouped kernel reads its pointers from device tables with vector loads: the
  // scalar operand of the load instructions needs them in scalar registers)
  auto scalar_ptr = [](const char* x) {
    const uint64_t v = (uint64_t)x;
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return (const char*)(((uint64_t)hi << 32) | lo);
  };
  // L2 prefetch (dense kernels without a K tail, whose buffer has the LDS this needs): the two LDS stages let a load
  // run at most one K step ahead of its use, about a microsecond - enough for operands that the last-level cache
  // holds, not for a first touch in HBM (after the reference's cache flush between timed calls every line is one).
  // So PFD K steps ahead of the loads each wave touches a few lines of the step to come: the 32 tiles that run on
  // one XCD at a time form a patch of 8 x 4, every A panel is shared by four of its programs and every B panel by
  // eight, and the programs split a panel's lines among themselves by their tile coordinates (tile column & 3 picks
  // the quarter of the A rows, tile row & 7 the eighth of the B rows), the four waves split that share again.  One
  // lane per 128-byte line, 16 + 8 lines per wave and K step.
  constexpr bool PF = XCD && !TAIL && MI355_W128_PREFETCH;
  constexpr int PFD = MI355_W128_PREFETCH_DISTANCE;
  const char* pA = nullptr;
  const char* pB = nullptr;
  unsigned voffPA = 0, voffPB = 0;
  if constexpr (PF) {
    voffPA = (lane % (BM / 16)) * (unsigned)p.lda;
    voffPB = B_KMAJOR ? (lane & 7) * (unsigned)p.ldb : ((lane & 7) >> 2) * (unsigned)p.ldb + (lane & 3) * 128;
  }
  auto set_fill_tile = [&](int fm, int fn) {
    fA = scalar_ptr(p.A + ((int64_t)fm * BM + wave * (BM / 4)) * p.lda);
    fB = scalar_ptr(B_KMAJOR ? p.B + ((int64_t)fn * BN + wave * 64) * p.ldb
                             : p.B + (int64_t)fn * BN * 2 + (int64_t)(wave * 16) * p.ldb);
    if constexpr (PF) {
      pA = scalar_ptr(p.A + ((int64_t)fm * BM + (fn & 3) * (BM / 4) + wave * (BM / 16)) * p.lda);
      pB = scalar_ptr(B_KMAJOR ? p.B + ((int64_t)fn * BN + (fm & 7) * 32 + wave * 8) * p.ldb
                               : p.B + (int64_t)fn * BN * 2 + (int64_t)((fm & 7) * 8 + wave * 2) * p.ldb);
    }
  };
  set_fill_tile(pm, pn);
  const unsigned kstepB = B_KMAJOR ? ROWB : 64 * (unsigned)p.ldb;   // bytes from one K step to the next
  // load j (0..7: A, 8..15: B) of the K step at (srcA, srcB) into the stage at `stage_base`.  M0 = middle of the
  // wave's 8 KiB of that operand, instruction offsets -4096 .. 3072.
  auto load_of = [](int slot) constexpr { return slot < LA ? slot : 8 + slot - LA; };   // load slot -> j (A: 0 .. LA-1, B: 8 .. 15)
  auto issue = [&](auto J_, const char* srcA, const char* srcB, unsigned stage_base, auto SETTLE_) {
    constexpr int j = decltype(J_)::value, q = j & 7, ioff = (q - 4) * 1024;
    const unsigned dst = stage_base + (j < 8 ? wave * (LA * 1024) : A_BYTES + wave * 8192) + 4096;
    if constexpr (j < 8) async_copy16_sbase_off<ioff, q == 0, decltype(SETTLE_)::value>(srcA, voffA[q], dst);
    else async_copy16_sbase_off<ioff, q == 0, decltype(SETTLE_)::value>(srcB, voffB[q], dst);
  };

  // ---- fragment reads: lane (l16, kg) of sub-step ks wants chunk 4 ks + kg of row l16 (+ 16 t)
  unsigned adrA[KS], adrB[B_KMAJOR ? KS : NT];   // stage 0; stage 1 is 64 KiB further (added at the read)
  {
    const unsigned s = (l16 >> 1) & 7;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      const unsigned slot = ((4 * ks + kg) ^ s) * 16;
      adrA[ks] = lds0 + (wm * (BM / 2) + l16) * ROWB + slot;
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
  static_for<NLOADS>([&](auto L_) { issue(std::integral_constant<int, load_of(decltype(L_)::value)>{}, fA, fB, lds0, std::true_type{}); });
  static_for<NLOADS>([&](auto L_) { issue(std::integral_constant<int, load_of(decltype(L_)::value)>{}, fA + ROWB, fB + kstepB, lds0 + STAGE, std::true_type{}); });
  fA += 2 * ROWB;
  fB += 2 * (int64_t)kstepB;
  if constexpr (PF) {
    // the lines of K steps 2 and 3 (the loop's touches begin with step 2 + PFD); also the two youngest loads that
    // the loop's waits leave outstanding from the first step on
    const int k2 = min(2, nk - 1), k3 = min(3, nk - 1);
    touch_line_sbase<true, BM / 16>(pA + k2 * ROWB, voffPA, lds0 + 2 * STAGE + wave * 256);
    touch_line_sbase<false, 8>(pB + (int64_t)k2 * kstepB, voffPB, 0u);
    touch_line_sbase<false, BM / 16>(pA + k3 * ROWB, voffPA, 0u);
    touch_line_sbase<false, 8>(pB + (int64_t)k3 * kstepB, voffPB, 0u);
    pA += 2 * ROWB;
    pB += 2 * (int64_t)kstepB;
  }
  wait_vmcnt<NLOADS + (PF ? 4 : 0)>();
  block_barrier();
  using Z = std::integral_constant<int, 0>;
  static_for<NRD>([&](auto OP_) { read_one(OP_, Z{}, Z{}, f[0]); });

  // One sub-step: 64 MFMAs on f[ks]; the fragments of the next sub-step are requested over the first
  // half of them (one read per two MFMAs).  The last sub-step of a stage first meets the other waves
  // (every wave has then read all it needs of this stage, and the other stage has landed), reads the
  // first fragments of the other stage and refills this one with the tile two steps ahead (one load
  // per four MFMAs).
  auto substep = [&](auto P_, auto KS_, auto MORE_, auto REFILL_, const char* tA, const char* tB) {
    constexpr int P = decltype(P_)::value, ks = decltype(KS_)::value, cur = ks & 1, nxt = cur ^ 1;
    constexpr bool last = ks == KS - 1;
    constexpr bool more = decltype(MORE_)::value;              // there is a next sub-step to read for
    constexpr bool refill = last && decltype(REFILL_)::value;  // and a tile two steps ahead to request
    lds_wait<0>();
    pin(f[cur]);
    if constexpr (last) {
      wait_vmcnt<PF ? 2 : 0>();   // (all but the two touches of the previous step, which are the youngest loads)
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
      constexpr int every = NM / 16;   // MFMAs per load slot: 4 (64 MFMAs) or 3 (48)
      if constexpr (refill && n % every == 1 && n / every < NLOADS)
        issue(std::integral_constant<int, load_of(n / every)>{}, fA, fB, lds0 + P * STAGE, std::false_type{});
      if constexpr (refill && PF && n == NM - 2) touch_line_sbase<true, BM / 16>(tA, voffPA, lds0 + 2 * STAGE + wave * 256);
      if constexpr (refill && PF && n == NM - 1) touch_line_sbase<false, 8>(tB, voffPB, 0u);
      if constexpr (n % 2 == 1) __builtin_amdgcn_sched_barrier(0);
    });
  };
  using I0 = std::integral_constant<int, 0>; using I1 = std::integral_constant<int, 1>;
  using T = std::true_type; using F = std::false_type;
  // A K step; its loads fetch the K step that the scalar bases point at.
  auto stage = [&](auto P_, const char* tA, const char* tB) {
    substep(P_, I0{}, T{}, F{}, tA, tB);
    substep(P_, I1{}, T{}, T{}, tA, tB);
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
  // the lines to touch: K step fk + PFD of the fill tile, or (past its end) the step being fetched anyway
  const int64_t pfdB = (int64_t)PFD * kstepB;
  auto touch_a = [&]() { return PF ? pA + (fk + PFD < nk ? PFD * ROWB : 0) : nullptr; };
  auto touch_b = [&]() { return PF ? pB + (fk + PFD < nk ? pfdB : (int64_t)0) : nullptr; };
  auto advance = [&]() {
    fA += ROWB;
    fB += kstepB;
    if constexpr (PF) { pA += ROWB; pB += kstepB; }
    if (++fk == nk) {
      fk = 0;
      if (ftile + tile_step < tend) ftile += tile_step;
      int fm, fn;
      tile_at(ftile, fm, fn);
      set_fill_tile(fm, fn);
    }
  };
  if (nk == 2) { fk = 1; advance(); }   // (two steps per tile: the prologue fetched both, the cursor is on the next tile)
  while (true) {
    // With the touches in flight the loop's waits leave two loads outstanding, and the compiler, which counts only
    // the loads IT knows, must then assume that the last two registers it reloaded behind the epilogue (lane offsets
    // of the loads, spilled there) are still on their way: it guarded their first use - inside the K loop - with a
    // wait for ALL outstanding loads, a full drain in every step (-6 to -12 %).  One full wait per tile in front of
    // the loop tells it that its reloads have landed; the stores of the epilogue are all that this waits for.
    if constexpr (PF) wait_all();
    for (int kt = 0; kt < nk; kt += 2) {
      stage(I0{}, touch_a(), touch_b()); advance();
      stage(I1{}, touch_a(), touch_b()); advance();
      if (kt + 2 >= nk_last) mfma_retire();
    }
    if constexpr (TAIL) {
      const int k_main = nk * ROWB, tail = p.k_bytes - k_main;   // bytes per row: done, and left (a multiple of 16)
      const unsigned tailA = lds0 + 2 * STAGE, tailB = tailA + BM * 64;
      const char* const tA = p.A + (int64_t)pm * BM * p.lda + k_main;
      for (int h = 0; h * 64 < tail; h++) {
        // this half-step's 64 bytes of the 256 A rows and of the 256 B rows (K-major B) or its 32 k rows of 512
        // bytes (row-major B, in the column-group order of the stages): 1024 + 1024 chunks of 16 bytes, four
        // each per thread, zeros beyond K
        i32x4 va[4], vb[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
          const int id = tid + 256 * i;
          {
            const int row = id >> 2, kb = h * 64 + (id & 3) * 16;
            va[i] = i32x4{0, 0, 0, 0};
            if (kb < tail) va[i] = *(const i32x4*)(tA + (int64_t)row * p.lda + kb);
          }
          vb[i] = i32x4{0, 0, 0, 0};
          if constexpr (B_KMAJOR) {
            const int row = id >> 2, kb = h * 64 + (id & 3) * 16;
            if (kb < tail) vb[i] = *(const i32x4*)(p.B + ((int64_t)pn * BN + row) * p.ldb + k_main + kb);
          } else {
            const int kr = id >> 5, pc = id & 31;
            const int k = k_main / 2 + h * 32 + kr;
            const int lg = (pc >> 1) ^ (2 * (kr & 3)) ^ ((kr >> 3) & 1);
            if (k < p.K) vb[i] = *(const i32x4*)(p.B + (int64_t)k * p.ldb + (int64_t)pn * BN * 2 + lg * 32 + (pc & 1) * 16);
          }
        }
#pragma unroll
        for (int i = 0; i < 4; i++) {
          const int id = tid + 256 * i;
          *(LDS_PTR(i32x4))(uintptr_t)(tailA + id * 16) = va[i];     // A: row id / 4 at 64 (id / 4), chunk id % 4
          *(LDS_PTR(i32x4))(uintptr_t)(tailB + id * 16) = vb[i];     // B: the same, or k row id / 32, chunk id % 32
        }
        lds_wait<0>();
        block_barrier();
        static_for<MT>([&](auto T_) {
          constexpr int t = decltype(T_)::value;
          f[1].a[t] = __builtin_bit_cast(V8, lds_read_b128<t * 16 * 64>(tailA + (wm * 128 + l16) * 64 + kg * 16));
        });
        static_for<NT>([&](auto T_) {
          constexpr int t = decltype(T_)::value;
          if constexpr (B_KMAJOR) {
            f[1].b[t] = __builtin_bit_cast(V8, lds_read_b128<t * 16 * 64>(tailB + (wn * 128 + l16) * 64 + kg * 16));
          } else {
            const unsigned ad = adrB[t] - (lds0 + A_BYTES) + tailB;
            s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_PTR(s16x4))(uintptr_t)ad);
            s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_PTR(s16x4))(uintptr_t)(ad + 4 * BN * 2));
            f[1].b[t] = __builtin_bit_cast(V8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
          }
        });
        lds_wait<0>();
        pin(f[1]);
        block_barrier();   // every wave holds its fragments: the buffer may be overwritten
        static_for<NM>([&](auto N_) {
          constexpr int n = decltype(N_)::value, i = n / NT, j = n % NT;
          mfma16(f[1].b[j], f[1].a[i], acc[i][j]);
        });
      }
      mfma_retire();
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
    int em = pm * BM + wm * (BM / 2), en = pn * BN + wn * 128, el = l16, ek = kg;
    asm volatile("" : "+s"(em), "+s"(en), "+v"(el), "+v"(ek));
    using OwnT = std::conditional_t<std::is_same<V8, bf16x8>::value, __bf16, _Float16>;
    if constexpr (EPI == 1) {
      // (the grouped GEMM: C rows of 16-byte alignment, as the reference's own groups have them, take the stores of
      // the lean epilogue - the scales are null pointers here)
      if (p.c_vec_ok && p.ldc % 8 == 0) gemm_epilogue16_lean<MT, NT, OwnT>(acc, p, em, en, el, ek);
      else gemm_epilogue16_plain<MT, NT, OwnT>(acc, p, em, en, el, ek);
    } else if constexpr (EPI == 3) gemm_epilogue16_lean<MT, NT, OwnT>(acc, p, em, en, el, ek);
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
template <typename V8, bool B_KMAJOR, int EPI, bool TAIL = false, int BM = 256>
__global__ __launch_bounds__(256, 1) void gemm_wave128_kernel(GemmArgs p) {
#if MI355_DEVICE_PASS
  extern __shared__ __attribute__((aligned(1024))) char lds_raw[];
  gemm_wave128_tiles<V8, B_KMAJOR, true, EPI, TAIL, BM>(p, blockIdx.x, gridDim.x, lds_addr((LDS_PTR(const void))lds_raw));
#endif
}

// Two tile heights in one launch, for tile counts that fill the last round of CUs badly and an M that is no multiple
// of 192: the first `rows256` rows of C on tiles of 256 x 256, the rows below on tiles of 192 x 256.  Every program walks
// its 256-row tiles (b, b + G, ...) and then its 192-row tiles, which are dealt from the other end (G - 1 - b, ...), so
// that the programs with one tile fewer in the first part are the ones with one more in the second; a program moves on
// by itself, nobody waits for the first part as a whole - which is what two launches would do.  5120^3 on 256 CUs: 400
// tiles are two rounds of which the second is 56 % full; 220 tiles of 256 rows + 240 of 192 are one tile of each per
// program.  (Lean epilogue, whole pairs of K steps: gemm_wave128_mixed_ok.)
template <typename V8, bool B_KMAJOR>
__global__ __launch_bounds__(256, 1) void gemm_wave128_mixed_kernel(GemmArgs p, int rows256) {
#if MI355_DEVICE_PASS
  extern __shared__ __attribute__((aligned(1024))) char lds_raw[];
  const unsigned lds0 = lds_addr((LDS_PTR(const void))lds_raw);
  const int G = gridDim.x, nn = p.N / 256;
  {
    GemmArgs q = p;
    q.M = rows256;
    if ((int)blockIdx.x < (rows256 / 256) * nn) gemm_wave128_tiles<V8, B_KMAJOR, true, 3, false, 256>(q, blockIdx.x, G, lds0);
  }
  // (every wave has waited for its own loads; the stages are laid out differently from here on, so no wave may
  // request its first loads of the second part while another's last loads of the first part could still land)
  block_barrier();
  {
    GemmArgs q = p;
    q.A = p.A + (int64_t)rows256 * p.lda;
    q.C = p.C + (int64_t)rows256 * p.ldc * 2;
    q.M = p.M - rows256;
    const int j = G - 1 - (int)blockIdx.x;
    if (j < (q.M / 192) * nn) gemm_wave128_tiles<V8, B_KMAJOR, true, 3, false, 192>(q, j, G, lds0);
  }
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
// kg and 4 + kg of its row (the lane group in the LOW bits of the chunk number: with 2 kg and 2 kg + 1, the
// first version, every ds_read_b128 took 8 instead of 4 cycles - LDS bank conflicts in half of the LDS cycles).  The fragment reads are ordinary LDS loads here (the compiler then
// places the two halves directly in the eight-register operand and waits for each fragment just
// before its first use); the direct global->LDS loads stay invisible to its bookkeeping.
// ---------------------------------------------------------------------------------------------
// The tail's fragments come from ordinary loads and moves that the compiler schedules; the MFMAs that read them are
// assembly it cannot see into: everything that writes these registers has completed behind this statement (the values
// pass through it) and two idle cycles separate the last such write from the first MFMA.
template <int NA, int NB>
__device__ __forceinline__ void settle_operands(i32x8 (&a)[NA], i32x8 (&b)[NB]) {
#if MI355_DEVICE_PASS
  static_assert(NA == 4 && NB == 8, "four A fragments and the first four of the B set");
  asm volatile("s_nop 1" : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]), "+v"(b[0]), "+v"(b[1]), "+v"(b[2]), "+v"(b[3]));
#endif
}

template <int FMT>
__device__ __forceinline__ void mfma16_f8(const i32x8& a, const i32x8& b, f32x4& c) {
#if MI355_DEVICE_PASS
  if constexpr (FMT == 0) asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
  else asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, %0 cbsz:1 blgp:1" : "+a"(c) : "v"(a), "v"(b));
#endif
}

// EPI: 0 = general epilogue, 2 = with the addend, 3 / 4 = lean epilogue writing fp16 / bf16
// TAIL: K bytes need not be a multiple of 256 (of 16 still): the main loop does the whole pairs of K steps, and what is
// left of each row (16 .. 240 bytes, the same for every tile) follows as one or two K steps whose fragments every lane
// loads straight from global memory - the same two chunks per 128-byte step as from LDS, zeros beyond K, the masked
// tail of the reference's loop (python/tutorials/03-matrix-multiplication.py:297-298) - into the fragment registers
// that the pipeline has free at that point (it already holds the next tile's first B and A fragments in the others).
// B_KMAJOR = false: B is row-major [K, N].  Its stage holds the K step's 128 k rows of 256 bytes (wave w loads the rows
// 32 w .. 32 w + 31, four per load); the 16-byte chunk c of row k lives in chunk c ^ g(k), g(k) = (k & 7) | 8 ((k >> 4) & 1),
// and a B fragment is four 8-bit transpose reads (ds_read_b64_tr_b8: within 16 lanes, lane 2 r + h addresses the bytes
// 8 h .. 8 h + 7 of row r, lane j receives column j of the 8 rows) of the rows 16 kg + {0, 8, 64, 72} + l16 / 2 - the K
// positions of the two chunks that the A fragment of the same lane group holds, in the same order.  g is the same for
// the four reads of a lane (they differ in bits 3 and 6 of k), so a fragment has one address and four immediates;
// the 8 rows x 2 chunks that a half-wave reads fall on 16 different bank groups.
// BM = 192: tiles of 192 x 256 (a wave: 96 x 128, six A fragments), for products whose 256 x 256 tiles fill the last
// round of CUs badly - as in the 16-bit kernel; lean epilogue, whole pairs of K steps.  BM = 128: tiles of 128 x 256 (a
// wave: 64 x 128, four A fragments; twelve loads for the sixteen MFMAs of a half step), for products with too few
// 256 x 256 tiles for this kernel.
// The calling workgroup computes the tiles `tile`, `tile + tile_step`, ... of the problem with the LDS at `lds_raw`.
template <int FMT, int EPI, bool TAIL = false, bool B_KMAJOR = true, int BM = 256>
__device__ __forceinline__ void gemm_wave128_f8_tiles(const GemmArgs& p, int tile, const int tile_step, LDS_PTR(char) const lds_raw) {
  static_assert(BM == 256 || ((BM == 192 || BM == 128) && !TAIL && (EPI == 3 || EPI == 4)), "192- and 128-row tiles: lean epilogue, no K tail");
  static_assert(B_KMAJOR || !TAIL, "the K tail loads K-contiguous fragments");
#if MI355_DEVICE_PASS
  constexpr int BN = 256, ROWB = 128;
  constexpr int A_BYTES = BM * ROWB, STAGE = A_BYTES + BN * ROWB;  // 64 KiB (56 KiB)
  constexpr int MT = BM / 32, NT = 8, MH = MT / 2;
  constexpr int LA = BM / 32, NLOADS = LA + 8;                      // direct loads per wave and K step: A, then B
  const unsigned lds0 = lds_addr((LDS_PTR(const void))lds_raw);

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int l16 = lane & 15, kg = lane >> 4;

  const int num_m = p.M / BM, num_n = p.N / BN;
  const int ntiles = num_m * num_n;
  int pm, pn;   // (the tiles are computed as one stream of K steps)
  grouped_tile(xcd_remap(tile, ntiles), num_m, num_n, p.group_m, pm, pn);
  const int nk = TAIL ? p.k_bytes / (2 * ROWB) * 2 : p.k_bytes / ROWB;
  int nk_last = nk;   // the same number, but opaque: see mfma_retire
  asm volatile("" : "+s"(nk_last));

  // ---- direct loads, exactly as in the 16-bit kernel (the tiles are the same bytes): a lane offset per load,
  // one scalar base per operand that moves with the K step being fetched
  const unsigned drow = lane >> 3, dslot = lane & 7;
  unsigned voffA[LA], voffB[8];
#pragma unroll
  for (int q = 0; q < 8; q++) {
    const unsigned chunk = dslot ^ (((q & 1) * 4 + (lane >> 4)) & 7);
    if (q < LA) voffA[q] = (drow + 8 * q) * (unsigned)p.lda + chunk * 16 - (unsigned)((q - 4) * 1024);
    if constexpr (B_KMAJOR) {
      voffB[q] = (drow + 8 * q) * (unsigned)p.ldb + chunk * 16 - (unsigned)((q - 4) * 1024);
    } else {
      // load q of the wave: k rows 4 q .. 4 q + 3 of its 32 (lane i: row i / 16, physical chunk i % 16)
      const unsigned kr = 4 * q + (lane >> 4), g = (kr & 7) | (((kr >> 4) & 1) << 3);
      voffB[q] = kr * (unsigned)p.ldb + (((lane & 15) ^ g) * 16) - (unsigned)((q - 4) * 1024);
    }
  }
  const int64_t kstepB = B_KMAJOR ? (int64_t)ROWB : (int64_t)ROWB * p.ldb;   // bytes from one K step of B to the next
  // scalar bases of the K step the loads are fetching (two K steps ahead of the MFMAs)
  const char* fA;
  const char* fB;
  // L2 touches two K steps ahead of the loads, as in the 16-bit kernel: the programs of an XCD's 8 x 4 patch of
  // tiles share out the lines of the panels they have in common
  constexpr bool PF = MI355_W128_PREFETCH;
  constexpr int PFD = MI355_W128_PREFETCH_DISTANCE;
  const char* pA = nullptr;
  const char* pB = nullptr;
  // (row-major B: the K step's 128 rows of 256 bytes are 256 lines, line L = half L & 1 of row L / 2)
  const unsigned voffPA = (lane % (BM / 16)) * (unsigned)p.lda;
  const unsigned voffPB = B_KMAJOR ? (lane & 7) * (unsigned)p.ldb : ((lane & 7) >> 1) * (unsigned)p.ldb + (lane & 1) * 128;
  auto set_fill_tile = [&](int fm, int fn) {
    fA = p.A + ((int64_t)fm * BM + wave * (BM / 4)) * p.lda;
    fB = B_KMAJOR ? p.B + ((int64_t)fn * BN + wave * 64) * p.ldb : p.B + (int64_t)fn * BN + (int64_t)(wave * 32) * p.ldb;
    if constexpr (PF) {
      pA = p.A + ((int64_t)fm * BM + (fn & 3) * (BM / 4) + wave * (BM / 16)) * p.lda;
      pB = B_KMAJOR ? p.B + ((int64_t)fn * BN + (fm & 7) * 32 + wave * 8) * p.ldb
                    : p.B + (int64_t)fn * BN + (int64_t)((fm & 7) * 16 + wave * 4) * p.ldb;
    }
  };
  set_fill_tile(pm, pn);
  auto load_of = [](int slot) constexpr { return slot < LA ? slot : 8 + slot - LA; };   // load slot -> j (A: 0 .. LA-1, B: 8 .. 15)
  auto issue = [&](auto J_, const char* srcA, const char* srcB, unsigned stage_base, auto SETTLE_) {
    constexpr int j = decltype(J_)::value, q = j & 7, ioff = (q - 4) * 1024;
    const unsigned dst = stage_base + (j < 8 ? wave * (LA * 1024) : A_BYTES + wave * 8192) + 4096;
    if constexpr (j < 8) async_copy16_sbase_off<ioff, q == 0, decltype(SETTLE_)::value>(srcA, voffA[q], dst);
    else async_copy16_sbase_off<ioff, q == 0, decltype(SETTLE_)::value>(srcB, voffB[q], dst);
  };

  // ---- fragment reads: lane (l16, kg) wants the chunks kg, 4 + kg of row l16 (+ 16 t)
  LDS_PTR(const char) fragA[2];
  LDS_PTR(const char) fragB[2];
  {
    const unsigned s = (l16 >> 1) & 7;
#pragma unroll
    for (int c = 0; c < 2; c++) {
      const unsigned slot = ((kg + 4 * c) ^ s) * 16;
      fragA[c] = (LDS_PTR(const char))lds_raw + (wm * (BM / 2) + l16) * ROWB + slot;
      fragB[c] = (LDS_PTR(const char))lds_raw + A_BYTES + (wn * 128 + l16) * ROWB + slot;
    }
  }
  auto read_frag = [&](LDS_PTR(const char) (&base)[2], int off) {
    i32x4 lo = *(LDS_PTR(const i32x4))(base[0] + off);
    i32x4 hi = *(LDS_PTR(const i32x4))(base[1] + off);
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  };
  // row-major B: the address of fragment 0 in stage 0; fragment t is the chunk index XOR t (t < 8 and the term of
  // wn, 8, touch different bits than each other, g any of them)
  unsigned trB = 0;
  if constexpr (!B_KMAJOR) {
    const unsigned kr = 16 * kg + (l16 >> 1), g = (kr & 7) | (((kr >> 4) & 1) << 3);
    trB = lds0 + A_BYTES + kr * BN + (((wn * 8) ^ g) << 4) + (l16 & 1) * 8;
  }
  auto read_b = [&](auto T_, auto SO_) {   // B fragment t of the stage at byte offset SO
    constexpr int t = decltype(T_)::value, so = decltype(SO_)::value;
    if constexpr (B_KMAJOR) {
      return read_frag(fragB, so + t * 16 * ROWB);
    } else {
      const unsigned ad = (trB ^ (unsigned)(t << 4)) + so;
      typedef int i32x2v __attribute__((ext_vector_type(2)));
      const i32x2v r0 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((LDS_PTR(i32x2v))(uintptr_t)ad);
      const i32x2v r1 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((LDS_PTR(i32x2v))(uintptr_t)(ad + 8 * BN));
      const i32x2v r2 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((LDS_PTR(i32x2v))(uintptr_t)(ad + 64 * BN));
      const i32x2v r3 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((LDS_PTR(i32x2v))(uintptr_t)(ad + 72 * BN));
      const i32x4 lo = __builtin_shufflevector(r0, r1, 0, 1, 2, 3), hi = __builtin_shufflevector(r2, r3, 0, 1, 2, 3);
      return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    }
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
  static_for<NLOADS>([&](auto L_) { issue(std::integral_constant<int, load_of(decltype(L_)::value)>{}, fA, fB, lds0, std::true_type{}); });
  static_for<NLOADS>([&](auto L_) { issue(std::integral_constant<int, load_of(decltype(L_)::value)>{}, fA + ROWB, fB + kstepB, lds0 + STAGE, std::true_type{}); });
  fA += 2 * ROWB;
  fB += 2 * kstepB;
  if constexpr (PF) {
    // the lines of K steps 2 and 3 (the loop's touches begin with step 2 + PFD); also the two youngest loads that
    // the loop's waits leave outstanding from the first step on
    const int k2 = min(2, nk - 1), k3 = min(3, nk - 1);
    touch_line_sbase<true, BM / 16>(pA + k2 * ROWB, voffPA, lds0 + 2 * STAGE + wave * 256);
    touch_line_sbase<false, 8>(pB + k2 * kstepB, voffPB, 0u);
    touch_line_sbase<false, BM / 16>(pA + k3 * ROWB, voffPA, 0u);
    touch_line_sbase<false, 8>(pB + k3 * kstepB, voffPB, 0u);
    pA += 2 * ROWB;
    pB += 2 * kstepB;
  }
  wait_vmcnt<NLOADS + (PF ? 4 : 0)>();
  block_barrier();
  static_for<NT>([&](auto T_) { b[0][decltype(T_)::value] = read_b(T_, std::integral_constant<int, 0>{}); });
#pragma unroll
  for (int t = 0; t < MH; t++) a0[t] = read_frag(fragA, t * 16 * ROWB);

  // One K step on stage P with the B fragments of set `cur`; its loads fetch the K step the scalar bases point at.
  auto step = [&](auto P_, auto CUR_, const char* tA, const char* tB) {
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
    wait_vmcnt<PF ? 2 : 0>();   // (all but the two touches of the previous step, which are the youngest loads)
    block_barrier();
    static_for<MH * NT>([&](auto N_) {
      constexpr int n = decltype(N_)::value, i = n / NT, j = n % NT;
      mfma16_f8<FMT>(b[cur][j], a1[i], acc[MH + i][j]);
      if constexpr (n < NT) b[nxt][n] = read_b(std::integral_constant<int, n>{}, std::integral_constant<int, sn>{});
      if constexpr (n >= NT && n < NT + MH) a0[n - NT] = read_frag(fragA, sn + (n - NT) * 16 * ROWB);
      // (one load per two MFMAs; the 192-row tile has 14 loads for its 24 MFMAs, the 128-row tile 12 for 16: from MFMA R
      // on every MFMA is followed by one.  The loads stay in slot order - A, then B - because only the first of each
      // operand sets M0.)
      constexpr int HALF = MH * NT, EXTRA = NLOADS > HALF / 2 ? NLOADS - HALF / 2 : 0, R = HALF - 2 * EXTRA;
      if constexpr (n < R && n % 2 == 1 && n / 2 < NLOADS) issue(std::integral_constant<int, load_of(n / 2)>{}, fA, fB, lds0 + P * STAGE, std::false_type{});
      if constexpr (n >= R) issue(std::integral_constant<int, load_of(R / 2 + n - R)>{}, fA, fB, lds0 + P * STAGE, std::false_type{});
      if constexpr (n % 2 == 1) __builtin_amdgcn_sched_barrier(0);
    });
    if constexpr (PF) {
      touch_line_sbase<true, BM / 16>(tA, voffPA, lds0 + 2 * STAGE + wave * 256);
      touch_line_sbase<false, 8>(tB, voffPB, 0u);
    }
  };
  using I0 = std::integral_constant<int, 0>; using I1 = std::integral_constant<int, 1>;
  // The fill cursor runs two K steps ahead of the MFMAs, across tile boundaries; behind the last tile it
  // wraps to that tile's first steps again (fetched into stages nobody reads any more), which keeps the
  // loop, the number of loads in flight and every wait uniform.
  int fk = 2, ftile = tile;
  // the lines to touch: K step fk + PFD of the fill tile, or (past its end) the step being fetched anyway
  auto touch_a = [&]() { return PF ? pA + (fk + PFD < nk ? PFD * ROWB : 0) : nullptr; };
  auto touch_b = [&]() { return PF ? pB + (fk + PFD < nk ? PFD * kstepB : (int64_t)0) : nullptr; };
  auto advance = [&]() {
    fA += ROWB;
    fB += kstepB;
    if constexpr (PF) { pA += ROWB; pB += kstepB; }
    if (++fk == nk) {
      fk = 0;
      if (ftile + tile_step < ntiles) ftile += tile_step;
      int fm, fn;
      grouped_tile(xcd_remap(ftile, ntiles), num_m, num_n, p.group_m, fm, fn);
      set_fill_tile(fm, fn);
    }
  };
  if (nk == 2) { fk = 1; advance(); }
  while (true) {
    if constexpr (PF) wait_all();   // (once per tile: tells the compiler that its own loads have landed, see the 16-bit kernel)
    for (int kt = 0; kt < nk; kt += 2) {
      step(I0{}, I0{}, touch_a(), touch_b()); advance();
      step(I1{}, I1{}, touch_a(), touch_b()); advance();
      if (kt + 2 >= nk_last) mfma_retire();
    }
    if constexpr (TAIL) {
      // (free here: a1 and the B set 1 - the last step read the next tile's first fragments into a0 and the B set 0)
      const int k_main = nk * ROWB, tail = p.k_bytes - k_main;
      int tm = pm * BM + wm * 128, tn = pn * BN + wn * 128, tl = l16, tk = kg;
      asm volatile("" : "+s"(tm), "+s"(tn), "+v"(tl), "+v"(tk));   // (keeps this address arithmetic out of the K loop)
      // a scalar base per fragment and one 32-bit lane offset per operand (gemm_wave128_f8_ok bounds 128 rows plus K)
      const char* const tA = p.A + (int64_t)tm * p.lda + k_main;
      const char* const tB = p.B + (int64_t)tn * p.ldb + k_main;
      const unsigned offA = (unsigned)tl * (unsigned)p.lda + tk * 16, offB = (unsigned)tl * (unsigned)p.ldb + tk * 16;
      for (int h = 0; h * ROWB < tail; h++) {
        const bool lo_ok = h * ROWB + tk * 16 < tail, hi_ok = h * ROWB + 64 + tk * 16 < tail;
        auto frag = [&](const char* src, unsigned off) {
          i32x4 lo = {0, 0, 0, 0}, hi = {0, 0, 0, 0};
          if (lo_ok) lo = *(const i32x4*)(src + h * ROWB + (uint64_t)off);
          if (hi_ok) hi = *(const i32x4*)(src + h * ROWB + 64 + (uint64_t)off);
          return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        };
        // (a quarter of the wave's tile at a time - four B and four A fragments: with all eight B fragments at once the
        // compiler spills lane offsets of the K loop across the tail and reloads them in front of the loop, behind
        // the wait there, so that their first use inside the loop would drain every load, in every step)
        static_for<4>([&](auto Q_) {
          constexpr int bh = decltype(Q_)::value / 2, ah = decltype(Q_)::value % 2;
          if constexpr (ah == 0) {
#pragma unroll
            for (int t = 0; t < MH; t++) b[1][t] = frag(tB + (int64_t)(bh * MH + t) * 16 * p.ldb, offB);
          }
#pragma unroll
          for (int t = 0; t < MH; t++) a1[t] = frag(tA + (int64_t)(ah * MH + t) * 16 * p.lda, offA);
          settle_operands(a1, b[1]);
          static_for<MH * MH>([&](auto N_) {
            constexpr int n = decltype(N_)::value, i = n / MH, j = n % MH;
            mfma16_f8<FMT>(b[1][j], a1[i], acc[ah * MH + i][bh * MH + j]);
          });
        });
        mfma_retire();   // (inside the loop's block, like the main loop's: see mfma_retire)
      }
    }
    mfma_drain(acc);
    int em = pm * BM + wm * (BM / 2), en = pn * BN + wn * 128, el = l16, ek = kg;
    asm volatile("" : "+s"(em), "+s"(en), "+v"(el), "+v"(ek));   // (keeps the epilogue's address arithmetic out of the K loop)
    if constexpr (EPI == 3) gemm_epilogue16_lean<MT, NT, _Float16>(acc, p, em, en, el, ek);
    else if constexpr (EPI == 4) gemm_epilogue16_lean<MT, NT, __bf16>(acc, p, em, en, el, ek);
    else gemm_epilogue16<MT, NT, EPI == 2>(acc, p, em, en, el, ek);
    tile += tile_step;
    if (tile >= ntiles) break;
    grouped_tile(xcd_remap(tile, ntiles), num_m, num_n, p.group_m, pm, pn);
    zero_acc();
  }
  wait_vmcnt<0>();  // nothing may still be writing LDS when the workgroup ends
#endif
}

// Workgroup b computes the tiles b, b + gridDim.x, ... (the grid: wave128_grid).
template <int FMT, int EPI, bool TAIL = false, bool B_KMAJOR = true, int BM = 256>
__global__ __launch_bounds__(256, 1) void gemm_wave128_f8_kernel(GemmArgs p) {
#if MI355_DEVICE_PASS
  extern __shared__ __attribute__((aligned(1024))) char lds_raw[];
  gemm_wave128_f8_tiles<FMT, EPI, TAIL, B_KMAJOR, BM>(p, blockIdx.x, gridDim.x, (LDS_PTR(char))lds_raw);
#endif
}

// Two tile heights in one launch, as gemm_wave128_mixed_kernel: the first `rows256` rows of C on tiles of 256 x 256, the
// rows below on tiles of 192 x 256 dealt from the other end of the grid (K-major B, lean epilogue, whole pairs of K steps).
template <int FMT, int EPI>
__global__ __launch_bounds__(256, 1) void gemm_wave128_f8_mixed_kernel(GemmArgs p, int rows256) {
#if MI355_DEVICE_PASS
  extern __shared__ __attribute__((aligned(1024))) char lds_raw[];
  const int G = gridDim.x, nn = p.N / 256;
  {
    GemmArgs q = p;
    q.M = rows256;
    if ((int)blockIdx.x < (rows256 / 256) * nn) gemm_wave128_f8_tiles<FMT, EPI, false, true, 256>(q, blockIdx.x, G, (LDS_PTR(char))lds_raw);
  }
  block_barrier();   // (the stages are laid out differently from here on: see gemm_wave128_mixed_kernel)
  {
    GemmArgs q = p;
    q.A = p.A + (int64_t)rows256 * p.lda;
    q.C = p.C + (int64_t)rows256 * p.ldc * 2;
    q.M = p.M - rows256;
    const int j = G - 1 - (int)blockIdx.x;
    if (j < (q.M / 192) * nn) gemm_wave128_f8_tiles<FMT, EPI, false, true, 192>(q, j, G, (LDS_PTR(char))lds_raw);
  }
#endif
}

template <int FMT, int EPI>
static int launch_wave128_f8_mixed(const GemmArgs& p, int rows256, hipStream_t stream) {
  constexpr int smem = 2 * (256 + 256) * 128 + 1024;
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)gemm_wave128_f8_mixed_kernel<FMT, EPI>, hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) return (int)e;
    attr_set = true;
  }
  const int grid = p.num_programs > 0 ? p.num_programs : 256;
  gemm_wave128_f8_mixed_kernel<FMT, EPI><<<dim3(grid), dim3(256), smem, stream>>>(p, rows256);
  return (int)hipGetLastError();
}

int gemm_wave128_f8_mixed_launch(const GemmArgs& p, int rows256, bool e5m2, hipStream_t stream) {
  if (lean_epilogue_type(p) == 1) return e5m2 ? launch_wave128_f8_mixed<1, 3>(p, rows256, stream) : launch_wave128_f8_mixed<0, 3>(p, rows256, stream);
  return e5m2 ? launch_wave128_f8_mixed<1, 4>(p, rows256, stream) : launch_wave128_f8_mixed<0, 4>(p, rows256, stream);
}

// fp8: the first `rows256` rows on 256-row tiles and the rest on 192-row tiles, under the conditions of the 192-row tiles
bool gemm_wave128_f8_mixed_ok(const GemmArgs& p, bool b_kmajor, int rows256) {
  if (!(rows256 > 0 && rows256 < p.M && rows256 % 256 == 0 && (p.M - rows256) % 192 == 0)) return false;
  if (!(b_kmajor && p.N % 256 == 0 && p.k_bytes % 256 == 0 && p.k_bytes >= 256)) return false;
  if (lean_epilogue_type(p) == 0) return false;
  return p.lda * 8 + p.k_bytes < (1ll << 31) && p.ldb * 8 + p.k_bytes < (1ll << 31);
}

template <int FMT, int EPI, bool TAIL = false, bool B_KMAJOR = true, int BM = 256>
static int launch_wave128_f8(const GemmArgs& p, hipStream_t stream) {
  constexpr int smem = 2 * (BM + 256) * 128 + 1024;   // (two stages and the 1 KiB that the L2 touches land in)
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)gemm_wave128_f8_kernel<FMT, EPI, TAIL, B_KMAJOR, BM>, hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) return (int)e;
    attr_set = true;
  }
  const int tiles = (p.M / BM) * (p.N / 256);
  const int grid = wave128_grid(tiles, p.num_programs);
  gemm_wave128_f8_kernel<FMT, EPI, TAIL, B_KMAJOR, BM><<<dim3(grid), dim3(256), smem, stream>>>(p);
  return (int)hipGetLastError();
}

int gemm_wave128_f8_launch(const GemmArgs& p, bool e5m2, bool b_kmajor, hipStream_t stream) {
  if (p.tile_m == 192) {   // (gemm_wave128_f8_192_ok: K-major B, lean epilogue, whole pairs of K steps)
    if (lean_epilogue_type(p) == 1) return e5m2 ? launch_wave128_f8<1, 3, false, true, 192>(p, stream) : launch_wave128_f8<0, 3, false, true, 192>(p, stream);
    return e5m2 ? launch_wave128_f8<1, 4, false, true, 192>(p, stream) : launch_wave128_f8<0, 4, false, true, 192>(p, stream);
  }
  if (p.tile_m == 128) {   // (the same conditions)
    if (lean_epilogue_type(p) == 1) return e5m2 ? launch_wave128_f8<1, 3, false, true, 128>(p, stream) : launch_wave128_f8<0, 3, false, true, 128>(p, stream);
    return e5m2 ? launch_wave128_f8<1, 4, false, true, 128>(p, stream) : launch_wave128_f8<0, 4, false, true, 128>(p, stream);
  }
  if (!b_kmajor) {   // (gemm_wave128_f8_ok: whole pairs of K steps, no addend)
    const int lean = lean_epilogue_type(p);
    if (lean == 1) return e5m2 ? launch_wave128_f8<1, 3, false, false>(p, stream) : launch_wave128_f8<0, 3, false, false>(p, stream);
    if (lean == 2) return e5m2 ? launch_wave128_f8<1, 4, false, false>(p, stream) : launch_wave128_f8<0, 4, false, false>(p, stream);
    return e5m2 ? launch_wave128_f8<1, 0, false, false>(p, stream) : launch_wave128_f8<0, 0, false, false>(p, stream);
  }
  if (p.k_bytes % 256 != 0) {   // (gemm_wave128_f8_ok: no addend then)
    const int lean = lean_epilogue_type(p);
    if (lean == 1) return e5m2 ? launch_wave128_f8<1, 3, true>(p, stream) : launch_wave128_f8<0, 3, true>(p, stream);
    if (lean == 2) return e5m2 ? launch_wave128_f8<1, 4, true>(p, stream) : launch_wave128_f8<0, 4, true>(p, stream);
    return e5m2 ? launch_wave128_f8<1, 0, true>(p, stream) : launch_wave128_f8<0, 0, true>(p, stream);
  }
  if (p.aux) return e5m2 ? launch_wave128_f8<1, 2>(p, stream) : launch_wave128_f8<0, 2>(p, stream);
  const int lean = lean_epilogue_type(p);
  if (lean == 1) return e5m2 ? launch_wave128_f8<1, 3>(p, stream) : launch_wave128_f8<0, 3>(p, stream);
  if (lean == 2) return e5m2 ? launch_wave128_f8<1, 4>(p, stream) : launch_wave128_f8<0, 4>(p, stream);
  return e5m2 ? launch_wave128_f8<1, 0>(p, stream) : launch_wave128_f8<0, 0>(p, stream);
}

// fp8: whole tiles, at least one pair of 128-byte K steps; with a K-major B, what is left behind the last pair is the
// TAIL form's, which exists without the addend
bool gemm_wave128_f8_ok(const GemmArgs& p, bool b_kmajor) {
  if (!(p.M % 256 == 0 && p.N % 256 == 0 && p.k_bytes % 16 == 0 && p.k_bytes >= 256)) return false;
  if (p.k_bytes % 256 != 0 && p.aux) return false;
  if (p.lda * 8 + p.k_bytes >= (1ll << 31)) return false;
  if (b_kmajor) return p.ldb * 8 + p.k_bytes < (1ll << 31);
  // row-major B: whole pairs of K steps, no addend; 32 rows plus a tile row within 32-bit lane offsets
  return p.k_bytes % 256 == 0 && !p.aux && p.ldb % 16 == 0 && p.ldb * 32 + 256 < (1ll << 32);
}

// fp8 on tiles of 192 x 256 (128 x 256): M a multiple of 192 (128), K-major B, whole pairs of K steps, a 16-bit C through
// the lean epilogue
bool gemm_wave128_f8_192_ok(const GemmArgs& p, bool b_kmajor, int tile_m) {
  if (!(b_kmajor && p.M % tile_m == 0 && p.N % 256 == 0 && p.k_bytes % 256 == 0 && p.k_bytes >= 256)) return false;
  if (lean_epilogue_type(p) == 0) return false;
  return p.lda * 8 + p.k_bytes < (1ll << 31) && p.ldb * 8 + p.k_bytes < (1ll << 31);
}

bool gemm_wave128_ok(const GemmArgs& p, bool b_kmajor, int in_dtype) {
  // whole tiles, at least one pair of 128-byte K steps (what is left behind the last pair: the TAIL form, which
  // exists for 16-bit operands with the lean epilogue - C in the operands' type - only), 32-bit lane offsets
  if (!(p.M % 256 == 0 && p.N % 256 == 0 && p.k_bytes % 16 == 0 && p.k_bytes >= 256)) return false;
  if (p.k_bytes % 256 != 0 && !((in_dtype == 0 || in_dtype == 1) && lean_epilogue_type(p) == in_dtype + 1)) return false;
  if (p.lda * 8 + p.k_bytes >= (1ll << 31)) return false;
  // (row-major B: the per-load XOR of the column group acts on the whole lane offset, so the row term
  // in it - a multiple of the pitch - must leave the bits of the 512-byte tile row alone)
  return b_kmajor ? p.ldb * 8 + p.k_bytes < (1ll << 31) : (p.ldb % 512 == 0 && (int64_t)p.K * p.ldb + 512 < (1ll << 31));
}

// The 192 x 256 tiles: M a multiple of 192, whole pairs of K steps, C in the operands' type through the lean epilogue
// (the one instantiation per type and B layout).  Worth it where the 256 x 256 tiles leave CUs idle in the last round:
// 3072^3 has 144 of those for 256 CUs and 192 of these.
bool gemm_wave128_192_ok(const GemmArgs& p, bool b_kmajor, int in_dtype, int tile_m) {
  if (!(p.M % tile_m == 0 && p.N % 256 == 0 && p.k_bytes % 256 == 0 && p.k_bytes >= 256)) return false;
  if (!((in_dtype == 0 || in_dtype == 1) && lean_epilogue_type(p) == in_dtype + 1)) return false;
  if (p.lda * 8 + p.k_bytes >= (1ll << 31)) return false;
  return b_kmajor ? p.ldb * 8 + p.k_bytes < (1ll << 31) : (p.ldb % 512 == 0 && (int64_t)p.K * p.ldb + 512 < (1ll << 31));
}

template <typename V8, bool B_KMAJOR, int EPI, bool TAIL = false, int BM = 256>
static int launch_wave128(const GemmArgs& p, hipStream_t stream) {
  constexpr int smem = 2 * (BM + 256) * 128 + (TAIL ? 2 * 256 * 64 : 1024);   // (with the tail buffer: all 160 KiB of the CU; without: 1 KiB that the L2 touches land in)
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)gemm_wave128_kernel<V8, B_KMAJOR, EPI, TAIL, BM>, hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) return (int)e;
    attr_set = true;
  }
  const int tiles = (p.M / BM) * (p.N / 256);
  const int grid = wave128_grid(tiles, p.num_programs);
  gemm_wave128_kernel<V8, B_KMAJOR, EPI, TAIL, BM><<<dim3(grid), dim3(256), smem, stream>>>(p);
  return (int)hipGetLastError();
}

template <typename V8, bool B_KMAJOR>
static int launch_wave128_mixed(const GemmArgs& p, int rows256, hipStream_t stream) {
  constexpr int smem = 2 * (256 + 256) * 128 + 1024;
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)gemm_wave128_mixed_kernel<V8, B_KMAJOR>, hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) return (int)e;
    attr_set = true;
  }
  const int grid = p.num_programs > 0 ? p.num_programs : 256;
  gemm_wave128_mixed_kernel<V8, B_KMAJOR><<<dim3(grid), dim3(256), smem, stream>>>(p, rows256);
  return (int)hipGetLastError();
}

int gemm_wave128_mixed_launch(const GemmArgs& p, int rows256, bool bf16, bool b_kmajor, hipStream_t stream) {
  if (bf16) return b_kmajor ? launch_wave128_mixed<bf16x8, true>(p, rows256, stream) : launch_wave128_mixed<bf16x8, false>(p, rows256, stream);
  return b_kmajor ? launch_wave128_mixed<f16x8, true>(p, rows256, stream) : launch_wave128_mixed<f16x8, false>(p, rows256, stream);
}

// the first `rows256` rows on 256-row tiles and the rest on 192-row tiles: both parts non-empty and whole, and what the
// 192-row tiles ask for (whole pairs of K steps, C in the operands' type through the lean epilogue)
bool gemm_wave128_mixed_ok(const GemmArgs& p, bool b_kmajor, int in_dtype, int rows256) {
  if (!(rows256 > 0 && rows256 < p.M && rows256 % 256 == 0 && (p.M - rows256) % 192 == 0)) return false;
  if (!(p.N % 256 == 0 && p.k_bytes % 256 == 0 && p.k_bytes >= 256)) return false;
  if (!((in_dtype == 0 || in_dtype == 1) && lean_epilogue_type(p) == in_dtype + 1)) return false;
  if (p.lda * 8 + p.k_bytes >= (1ll << 31)) return false;
  return b_kmajor ? p.ldb * 8 + p.k_bytes < (1ll << 31) : (p.ldb % 512 == 0 && (int64_t)p.K * p.ldb + 512 < (1ll << 31));
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

template <typename V8>
static int gemm_wave128_launch_typed(const GemmArgs& p, bool b_kmajor, bool own_type_lean, hipStream_t stream) {
  if (p.tile_m == 192)   // (gemm_wave128_192_ok: whole K steps, the lean epilogue)
    return b_kmajor ? launch_wave128<V8, true, 3, false, 192>(p, stream) : launch_wave128<V8, false, 3, false, 192>(p, stream);
  if (p.tile_m == 128)
    return b_kmajor ? launch_wave128<V8, true, 3, false, 128>(p, stream) : launch_wave128<V8, false, 3, false, 128>(p, stream);
  if (p.k_bytes % 256 != 0)   // (gemm_wave128_ok: the lean epilogue then)
    return b_kmajor ? launch_wave128<V8, true, 3, true>(p, stream) : launch_wave128<V8, false, 3, true>(p, stream);
  if (p.aux) return b_kmajor ? launch_wave128<V8, true, 2>(p, stream) : launch_wave128<V8, false, 2>(p, stream);
  if (own_type_lean) return b_kmajor ? launch_wave128<V8, true, 3>(p, stream) : launch_wave128<V8, false, 3>(p, stream);
  return b_kmajor ? launch_wave128<V8, true, 0>(p, stream) : launch_wave128<V8, false, 0>(p, stream);
}

int gemm_wave128_launch(const GemmArgs& p, bool bf16, bool b_kmajor, hipStream_t stream) {
  const bool own_type_lean = lean_epilogue_type(p) == (bf16 ? 2 : 1);   // lean epilogue, C in the operands' type
  return bf16 ? gemm_wave128_launch_typed<bf16x8>(p, b_kmajor, own_type_lean, stream)
              : gemm_wave128_launch_typed<f16x8>(p, b_kmajor, own_type_lean, stream);
}

}  // namespace mi355

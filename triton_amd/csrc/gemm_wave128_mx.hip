// Block-scaled (MXFP8 / MXFP4) forms of the four-wave GEMM of gemm_wave128.hip: the same skeleton - one workgroup
// per 256x256 tile of C, four waves of 128x128 from 16x16 MFMAs, 128 bytes of every operand row per K step, two
// 64 KiB LDS stages filled by direct global->LDS loads with fixed scalar bases - with scaled 16x16x128 f8f6f4
// MFMAs and the e8m0 block scales travelling through a small LDS ring of their own.
#include "gemm_wave128.h"

namespace mi355 {

// Scaled fp8 (e4m3) MFMA with the accumulator pinned to the accumulation registers; byte 0 of the scale dwords.
__device__ __forceinline__ void mfma16_mxfp8(const i32x8& a, const i32x8& b, f32x4& c, int sa, int sb) {
#if MI355_DEVICE_PASS
  asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel_hi:[0,0,0]"
               : "+a"(c) : "v"(a), "v"(b), "v"(sa), "v"(sb));
#endif
}
// The tails' fragments and scales come from ordinary loads and moves that the compiler schedules; the MFMAs that read
// them are assembly it cannot see into: everything that writes these registers has completed behind this statement (the
// values pass through it) and two idle cycles separate the last such write from the first MFMA.
template <typename R>
__device__ __forceinline__ void settle_one(R& r) {
#if MI355_DEVICE_PASS
  asm volatile("" : "+v"(r));
#endif
}
template <typename... R>
__device__ __forceinline__ void settle_pass(R&... r) {
  (settle_one(r), ...);
}
template <typename... R>
__device__ __forceinline__ void settle_tail(R&... r) {
#if MI355_DEVICE_PASS
  settle_pass(r...);
  asm volatile("s_nop 1" ::: "memory");
  settle_pass(r...);
#endif
}
#ifndef MXFP8_CHUNK
#define MXFP8_CHUNK(kg, c) ((kg) + 4 * (c))
#endif

// MXFP8 (e4m3 codes, one e8m0 scale per 32 elements): the fp8 kernel above with scaled MFMAs; a K step is
// 128 elements = four scale blocks, the scales travel 16 bytes per row (four K steps) per direct load into a
// two-slot LDS ring like those of the MXFP4 kernel below.
// EPI: 0 = general epilogue, 3 / 4 = lean epilogue (gemm_epilogue16_lean) writing fp16 / bf16
// TAIL: K need not be a multiple of 1024 (of 32 still, the scale block): the main loop does the whole groups of eight K
// steps, and what is left of each row (32 .. 992 bytes, the same for every tile) follows in K steps whose fragments and
// scale bytes every lane loads straight from global memory - zeros (and the scale 1) beyond K - into the registers that
// the pipeline has free at that point, a quarter of the wave's tile at a time.
// BM = 192: tiles of 192 x 256, as in the MXFP4 kernel below.
template <int EPI, bool TAIL = false, int BM = 256>
__device__ __forceinline__ void gemm_wave128_mxfp8_tiles(const GemmArgs& p, int tile, const int tile_step, LDS_PTR(char) const lds_raw) {
  static_assert(BM == 256 || ((BM == 192 || BM == 128) && !TAIL && (EPI == 3 || EPI == 4)), "192- and 128-row tiles: lean epilogue, no K tail");
#if MI355_DEVICE_PASS
  constexpr int BN = 256, ROWB = 128;
  constexpr int A_BYTES = BM * ROWB, STAGE = A_BYTES + BN * ROWB;  // 64 KiB (56 KiB)
  constexpr int MT = BM / 32, NT = 8, MH = MT / 2;
  constexpr int LA = BM / 32, NLOADS = LA + 8;                      // direct loads per wave and K step: A, then B
  constexpr int SC_BASE = 2 * STAGE, SC_SLOT = (256 + BN) * 16;     // scale ring behind the two stages (A part: room for 256 rows)
  const unsigned lds0 = lds_addr((LDS_PTR(const void))lds_raw);

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int l16 = lane & 15, kg = lane >> 4;

  const int num_m = p.M / BM, num_n = p.N / BN;
  const int ntiles = num_m * num_n;
  int pm, pn;   // (the tiles tile, tile + tile_step, ... are computed as one stream of K steps)
  grouped_tile(xcd_remap(tile, ntiles), num_m, num_n, p.group_m, pm, pn);
  const int nk = TAIL ? p.k_bytes / (8 * ROWB) * 8 : p.k_bytes / ROWB;
  int nk_last = nk;   // the same number, but opaque: see mfma_retire
  asm volatile("" : "+s"(nk_last));

  // ---- direct loads, exactly as in the 16-bit kernel (the tiles are the same bytes)
  // (a lane offset per load - row, chunk, and the instruction offset taken back out - and one scalar base per
  // operand that moves with the K step being fetched)
  const unsigned drow = lane >> 3, dslot = lane & 7;
  unsigned voffA[LA], voffB[8];
#pragma unroll
  for (int q = 0; q < 8; q++) {
    const unsigned chunk = dslot ^ (((q & 1) * 4 + (lane >> 4)) & 7);
    if (q < LA) voffA[q] = (drow + 8 * q) * (unsigned)p.lda + chunk * 16 - (unsigned)((q - 4) * 1024);
    voffB[q] = (drow + 8 * q) * (unsigned)p.ldb + chunk * 16 - (unsigned)((q - 4) * 1024);
  }
  // scalar bases of the tile the loads are fetching (two K steps ahead of the MFMAs)
  const char* fA;   // operands: the K step being fetched
  const char* fB;
  const char* gSA;
  const char* gSB;
  // L2 touches two K steps ahead of the loads, as in the 16-bit kernel: the programs of an XCD's 8 x 4 patch of
  // tiles share out the lines of the panels they have in common
  constexpr bool PF = MI355_W128_PREFETCH;
  constexpr int PFD = MI355_W128_PREFETCH_DISTANCE;
  const char* pA = nullptr;
  const char* pB = nullptr;
  const unsigned voffPA = (lane % (BM / 16)) * (unsigned)p.lda, voffPB = (lane & 7) * (unsigned)p.ldb;
  const unsigned touch_lds = lds0 + SC_BASE + 2 * SC_SLOT + wave * 256;
  auto set_fill_tile = [&](int fm, int fn) {
    fA = p.A + ((int64_t)fm * BM + wave * (BM / 4)) * p.lda;
    fB = p.B + ((int64_t)fn * BN + wave * 64) * p.ldb;
    if constexpr (PF) {
      pA = p.A + ((int64_t)fm * BM + (fn & 3) * (BM / 4) + wave * (BM / 16)) * p.lda;
      pB = p.B + ((int64_t)fn * BN + (fm & 7) * 32 + wave * 8) * p.ldb;
    }
    gSA = (const char*)p.sA + ((int64_t)fm * BM + wave * (BM / 4)) * p.lds_a;
    gSB = (const char*)p.sB + ((int64_t)fn * BN + wave * 64) * p.lds_b;
  };
  set_fill_tile(pm, pn);
  auto load_of = [](int slot) constexpr { return slot < LA ? slot : 8 + slot - LA; };   // load slot -> j (A: 0 .. LA-1, B: 8 .. 15)
  auto issue = [&](auto J_, const char* srcA, const char* srcB, unsigned stage_base, auto SETTLE_) {
    constexpr int j = decltype(J_)::value, q = j & 7, ioff = (q - 4) * 1024;
    const unsigned dst = stage_base + (j < 8 ? wave * (LA * 1024) : A_BYTES + wave * 8192) + 4096;
    if constexpr (j < 8) async_copy16_sbase_off<ioff, q == 0, decltype(SETTLE_)::value>(srcA, voffA[q], dst);
    else async_copy16_sbase_off<ioff, q == 0, decltype(SETTLE_)::value>(srcB, voffB[q], dst);
  };

  // ---- scale loads: wave w fetches the 16 scale bytes (four K steps) of rows 64 w .. 64 w + 63 of A and of B
  const unsigned voffSA = lane * (unsigned)p.lds_a, voffSB = lane * (unsigned)p.lds_b;
  auto issue_scales = [&](int g, auto SETTLE_) {   // group g of four K steps of the fill tile -> slot g & 1 (K steps come in eights)
    const unsigned slot = lds0 + SC_BASE + (g & 1) * SC_SLOT;
    // (192-row tiles: a wave fetches the scales of its 48 A rows, the lanes beyond sit the load out)
    if (BM == 256 || lane < BM / 4) async_copy16_sbase<decltype(SETTLE_)::value>(gSA, voffSA + (unsigned)g * 16, slot + wave * (BM / 4) * 16);
    async_copy16_sbase<decltype(SETTLE_)::value>(gSB, voffSB + (unsigned)g * 16, slot + 256 * 16 + wave * 1024);
  };
  // scales of a K step: lane group kg supplies block kg of its row, fetched as one byte (ds_read_u8: it arrives in
  // byte 0, the position the MFMA's selector names, so no shift), one read per two MFMAs
  const unsigned adrSA = lds0 + SC_BASE + (wm * (BM / 2) + l16) * 16 + kg;
  const unsigned adrSB = lds0 + SC_BASE + 256 * 16 + (wn * 128 + l16) * 16 + kg;
  int sa[2][MT], sb[2][NT];
  auto read_scale = [&](auto OP_, auto SET_, auto OFF_) {   // OFF: slot * SC_SLOT + (K step & 3) * 4
    constexpr int op = decltype(OP_)::value, set = decltype(SET_)::value, off = decltype(OFF_)::value;
    if constexpr (op < MT) sa[set][op] = lds_read_u8<off + op * 256>(adrSA);
    else sb[set][op - MT] = lds_read_u8<off + (op - MT) * 256>(adrSB);
  };
  auto pin_scales = [&](auto SET_) {
    constexpr int set = decltype(SET_)::value;
    static_for<MT>([&](auto T_) { lds_use(sa[set][decltype(T_)::value]); });
    static_for<NT>([&](auto T_) { lds_use(sb[set][decltype(T_)::value]); });
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
      fragA[c] = (LDS_PTR(const char))lds_raw + (wm * (BM / 2) + l16) * ROWB + slot;
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
  issue_scales(0, std::true_type{});
  static_for<NLOADS>([&](auto L_) { issue(std::integral_constant<int, load_of(decltype(L_)::value)>{}, fA, fB, lds0, std::true_type{}); });
  static_for<NLOADS>([&](auto L_) { issue(std::integral_constant<int, load_of(decltype(L_)::value)>{}, fA + ROWB, fB + ROWB, lds0 + STAGE, std::true_type{}); });
  fA += 2 * ROWB;
  fB += 2 * ROWB;
  if constexpr (PF) {
    // the lines of K steps 2 and 3 (the loop's touches begin with step 2 + PFD); also the two youngest loads that
    // the loop's waits leave outstanding from the first step on
    const int k2 = min(2, nk - 1), k3 = min(3, nk - 1);
    touch_line_sbase<true, BM / 16>(pA + k2 * ROWB, voffPA, touch_lds);
    touch_line_sbase<false, 8>(pB + k2 * ROWB, voffPB, 0u);
    touch_line_sbase<false, BM / 16>(pA + k3 * ROWB, voffPA, 0u);
    touch_line_sbase<false, 8>(pB + k3 * ROWB, voffPB, 0u);
    pA += 2 * ROWB;
    pB += 2 * ROWB;
  }
  wait_vmcnt<NLOADS + (PF ? 4 : 0)>();
  block_barrier();
  static_for<MT + NT>([&](auto OP_) { read_scale(OP_, std::integral_constant<int, 0>{}, std::integral_constant<int, 0>{}); });
  lds_wait<0>();
  pin_scales(std::integral_constant<int, 0>{});
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
    wait_vmcnt<PF ? 2 : 0>();   // (all but the two touches of the previous step, which are the youngest loads)
    block_barrier();
    static_for<MH * NT>([&](auto N_) {
      constexpr int n = decltype(N_)::value, i = n / NT, j = n % NT;
      mfma16_mxfp8(b[cur][j], a1[i], acc[MH + i][j], sb[cur][j], sa[cur][MH + i]);
      if constexpr (n < NT) b[nxt][n] = read_frag(fragB, sn + n * 16 * ROWB);
      if constexpr (n >= NT && n < NT + MH) a0[n - NT] = read_frag(fragA, sn + (n - NT) * 16 * ROWB);
      // (the next step's scales: one read per two MFMAs, or - 192-row tiles, 14 reads for 24 MFMAs - one per MFMA)
      constexpr int HALF = MH * NT, NSC = MT + NT, EXTRA = NLOADS > HALF / 2 ? NLOADS - HALF / 2 : 0;
      using OffNext = std::integral_constant<int, (UN >> 2) * SC_SLOT + (UN & 3) * 4>;
      if constexpr (HALF >= 2 * NSC) {
        if constexpr (n % 2 == 0) read_scale(std::integral_constant<int, n / 2>{}, std::integral_constant<int, nxt>{}, OffNext{});
      } else {
        if constexpr (n < NSC) read_scale(std::integral_constant<int, n>{}, std::integral_constant<int, nxt>{}, OffNext{});
      }
      // (the scales of the K steps fk .. fk + 3 are requested in the third step of every four, into the slot whose
      // last reader was the read for the step before this one)
      // (between the last A load and the first B load, which sets M0 for its group again)
      if constexpr ((U & 3) == 2 && n == 2 * LA) issue_scales(fk >> 2, std::false_type{});
      // (one load per two MFMAs; the 192-row tile has 14 loads for its 24 MFMAs, the 128-row tile 12 for 16: from MFMA R
      // on every MFMA is followed by one.  The loads stay in slot order - A, then B - because only the first of each
      // operand sets M0.)
      constexpr int R = HALF - 2 * EXTRA;
      if constexpr (n < R && n % 2 == 1 && n / 2 < NLOADS) issue(std::integral_constant<int, load_of(n / 2)>{}, fA, fB, lds0 + P * STAGE, std::false_type{});
      if constexpr (n >= R) issue(std::integral_constant<int, load_of(R / 2 + n - R)>{}, fA, fB, lds0 + P * STAGE, std::false_type{});
      if constexpr (n % 2 == 1) __builtin_amdgcn_sched_barrier(0);
    });
    if constexpr (PF) {
      touch_line_sbase<true, BM / 16>(pA + (fk + PFD < nk ? PFD * ROWB : 0), voffPA, touch_lds);
      touch_line_sbase<false, 8>(pB + (fk + PFD < nk ? PFD * ROWB : 0), voffPB, 0u);
    }
    lds_wait<0>();
    pin_scales(std::integral_constant<int, nxt>{});
  };
  using I0 = std::integral_constant<int, 0>; using I1 = std::integral_constant<int, 1>;
  // The fill cursor runs two K steps ahead of the MFMAs, across tile boundaries; behind the last tile it
  // wraps to that tile's first steps again (fetched into stages nobody reads any more), which keeps the
  // loop, the number of loads in flight and every wait uniform.
  int fk = 2, ftile = tile;
  auto advance = [&]() {
    fA += ROWB;
    fB += ROWB;
    if constexpr (PF) { pA += ROWB; pB += ROWB; }
    if (++fk == nk) {
      fk = 0;
      if (ftile + tile_step < ntiles) ftile += tile_step;
      int fm, fn;
      grouped_tile(xcd_remap(ftile, ntiles), num_m, num_n, p.group_m, fm, fn);
      set_fill_tile(fm, fn);
    }
  };
  while (true) {
    if constexpr (PF) wait_all();   // (once per tile: tells the compiler that its own loads have landed, see the 16-bit kernel)
    for (int kt = 0; kt < nk; kt += 8) {
      static_for<8>([&](auto U_) { step(U_, fk); advance(); });
      if (kt + 8 >= nk_last) mfma_retire();
    }
    if constexpr (TAIL) {
      // (free here: a1, the B set 1 and the scale set 1 - the last step read the next tile's first fragments and scales
      // into the others)
      const int k_main = nk * ROWB, tail = p.k_bytes - k_main;
      int tm = pm * BM + wm * 128, tn = pn * BN + wn * 128, tl = l16, tk = kg;
      asm volatile("" : "+s"(tm), "+s"(tn), "+v"(tl), "+v"(tk));   // (keeps this address arithmetic out of the K loop)
      // a scalar base per fragment and one 32-bit lane offset per operand (gemm_wave128_mxfp8_ok bounds them)
      const char* const tA = p.A + (int64_t)tm * p.lda + k_main;
      const char* const tB = p.B + (int64_t)tn * p.ldb + k_main;
      const uint8_t* const tSA = p.sA + (int64_t)tm * p.lds_a + k_main / 32;
      const uint8_t* const tSB = p.sB + (int64_t)tn * p.lds_b + k_main / 32;
      unsigned offA = (unsigned)tl * (unsigned)p.lda + tk * 16, offB = (unsigned)tl * (unsigned)p.ldb + tk * 16;
      unsigned offSA = (unsigned)tl * (unsigned)p.lds_a + tk, offSB = (unsigned)tl * (unsigned)p.lds_b + tk;
      for (int h = 0; h * ROWB < tail; h++) {
        // chunk tk (low registers) and chunk 4 + tk (high registers) of the step; the scale of its block tk
        const bool lo_ok = h * ROWB + tk * 16 < tail, hi_ok = h * ROWB + 64 + tk * 16 < tail, sc_ok = h * ROWB + tk * 32 < tail;
        auto frag = [&](const char* src, unsigned off) {
          i32x4 lo = {0, 0, 0, 0}, hi = {0, 0, 0, 0};
          if (lo_ok) lo = *(const i32x4*)(src + h * ROWB + (uint64_t)off);
          if (hi_ok) hi = *(const i32x4*)(src + h * ROWB + 64 + (uint64_t)off);
          return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        };
        auto scale = [&](const uint8_t* src, unsigned off) {
          int v = 127;   // (2^0: multiplies zeros)
          if (sc_ok) v = src[h * 4 + (uint64_t)off];
          return v;
        };
        static_for<4>([&](auto Q_) {
          constexpr int bh = decltype(Q_)::value / 2, ah = decltype(Q_)::value % 2;
          // (the offsets pass through an assembly statement, which stays behind the MFMAs of the quarter before: the
          // compiler cannot start this quarter's loads earlier and so needs no second set of registers for them)
          asm volatile("" : "+v"(offA), "+v"(offB), "+v"(offSA), "+v"(offSB));
          if constexpr (ah == 0) {
#pragma unroll
            for (int t = 0; t < MH; t++) {
              b[1][t] = frag(tB + (int64_t)(bh * MH + t) * 16 * p.ldb, offB);
              sb[1][t] = scale(tSB + (int64_t)(bh * MH + t) * 16 * p.lds_b, offSB);
            }
          }
#pragma unroll
          for (int t = 0; t < MH; t++) {
            a1[t] = frag(tA + (int64_t)(ah * MH + t) * 16 * p.lda, offA);
            sa[1][t] = scale(tSA + (int64_t)(ah * MH + t) * 16 * p.lds_a, offSA);
          }
          settle_tail(a1[0], a1[1], a1[2], a1[3], b[1][0], b[1][1], b[1][2], b[1][3],
                      sa[1][0], sa[1][1], sa[1][2], sa[1][3], sb[1][0], sb[1][1], sb[1][2], sb[1][3]);
          static_for<MH * MH>([&](auto N_) {
            constexpr int n = decltype(N_)::value, i = n / MH, j = n % MH;
            mfma16_mxfp8(b[1][j], a1[i], acc[ah * MH + i][bh * MH + j], sb[1][j], sa[1][i]);
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
    else gemm_epilogue16<MT, NT>(acc, p, em, en, el, ek);
    tile += tile_step;
    if (tile >= ntiles) break;
    grouped_tile(xcd_remap(tile, ntiles), num_m, num_n, p.group_m, pm, pn);
    zero_acc();
  }
  wait_vmcnt<0>();  // nothing may still be writing LDS when the workgroup ends
#endif
}

// Workgroup b computes the tiles b, b + gridDim.x, ... (the grid: wave128_grid).
template <int EPI, bool TAIL = false, int BM = 256>
__global__ __launch_bounds__(256, 1) void gemm_wave128_mxfp8_kernel(GemmArgs p) {
#if MI355_DEVICE_PASS
  extern __shared__ __attribute__((aligned(1024))) char lds_raw[];
  gemm_wave128_mxfp8_tiles<EPI, TAIL, BM>(p, blockIdx.x, gridDim.x, (LDS_PTR(char))lds_raw);
#endif
}

// Two tile heights in one launch, as for the 16-bit and fp8 products: the first `rows256` rows of C on tiles of 256 x 256,
// the rows below (their operand and scale rows) on tiles of 192 x 256 dealt from the other end of the grid.
template <int EPI>
__global__ __launch_bounds__(256, 1) void gemm_wave128_mxfp8_mixed_kernel(GemmArgs p, int rows256) {
#if MI355_DEVICE_PASS
  extern __shared__ __attribute__((aligned(1024))) char lds_raw[];
  const int G = gridDim.x, nn = p.N / 256;
  {
    GemmArgs q = p;
    q.M = rows256;
    if ((int)blockIdx.x < (rows256 / 256) * nn) gemm_wave128_mxfp8_tiles<EPI, false, 256>(q, blockIdx.x, G, (LDS_PTR(char))lds_raw);
  }
  block_barrier();   // (the stages are laid out differently from here on; every wave has waited for its own loads)
  {
    GemmArgs q = p;
    q.A = p.A + (int64_t)rows256 * p.lda;
    q.sA = p.sA + (int64_t)rows256 * p.lds_a;
    q.C = p.C + (int64_t)rows256 * p.ldc * 2;
    q.M = p.M - rows256;
    const int j = G - 1 - (int)blockIdx.x;
    if (j < (q.M / 192) * nn) gemm_wave128_mxfp8_tiles<EPI, false, 192>(q, j, G, (LDS_PTR(char))lds_raw);
  }
#endif
}

template <int EPI>
static int launch_wave128_mxfp8_mixed(const GemmArgs& p, int rows256, hipStream_t stream) {
  constexpr int smem = 2 * (256 + 256) * 128 + 2 * 512 * 16 + 1024;
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)gemm_wave128_mxfp8_mixed_kernel<EPI>, hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) return (int)e;
    attr_set = true;
  }
  const int grid = p.num_programs > 0 ? p.num_programs : 256;
  gemm_wave128_mxfp8_mixed_kernel<EPI><<<dim3(grid), dim3(256), smem, stream>>>(p, rows256);
  return (int)hipGetLastError();
}

bool gemm_wave128_mxfp8_ok(const GemmArgs& p) {
  // whole tiles, at least one group of eight K steps (K >= 1024; what is left behind the last group: the TAIL form),
  // scale rows that a 16-byte load can fetch
  return p.M % 256 == 0 && p.N % 256 == 0 && p.k_bytes % 32 == 0 && p.k_bytes >= 1024 &&
         p.lda * 8 + p.k_bytes < (1ll << 31) && p.ldb * 8 + p.k_bytes < (1ll << 31) &&
         p.lds_a % 16 == 0 && p.lds_b % 16 == 0 && ((uintptr_t)p.sA | (uintptr_t)p.sB) % 16 == 0 &&
         p.lds_a * 64 + p.k_bytes / 32 < (1ll << 31) && p.lds_b * 64 + p.k_bytes / 32 < (1ll << 31);
}

template <int EPI, bool TAIL = false, int BM = 256>
static int launch_wave128_mxfp8(const GemmArgs& p, hipStream_t stream) {
  constexpr int smem = 2 * (BM + 256) * 128 + 2 * 512 * 16 + 1024;   // (stages, scale ring and the 1 KiB that the L2 touches land in)
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)gemm_wave128_mxfp8_kernel<EPI, TAIL, BM>, hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) return (int)e;
    attr_set = true;
  }
  const int tiles = (p.M / BM) * (p.N / 256);
  const int grid = wave128_grid(tiles, p.num_programs);
  gemm_wave128_mxfp8_kernel<EPI, TAIL, BM><<<dim3(grid), dim3(256), smem, stream>>>(p);
  return (int)hipGetLastError();
}

int gemm_wave128_mxfp8_launch(const GemmArgs& p, hipStream_t stream) {
  const int lean = lean_epilogue_type(p);
  if (p.tile_m == 192)   // (gemm_wave128_mx_192_ok: lean epilogue, whole groups of K steps)
    return lean == 1 ? launch_wave128_mxfp8<3, false, 192>(p, stream) : launch_wave128_mxfp8<4, false, 192>(p, stream);
  if (p.tile_m == 128)
    return lean == 1 ? launch_wave128_mxfp8<3, false, 128>(p, stream) : launch_wave128_mxfp8<4, false, 128>(p, stream);
  if (p.k_bytes % 1024 != 0)
    return lean == 1 ? launch_wave128_mxfp8<3, true>(p, stream) : lean == 2 ? launch_wave128_mxfp8<4, true>(p, stream) : launch_wave128_mxfp8<0, true>(p, stream);
  return lean == 1 ? launch_wave128_mxfp8<3>(p, stream) : lean == 2 ? launch_wave128_mxfp8<4>(p, stream) : launch_wave128_mxfp8<0>(p, stream);
}

// ---------------------------------------------------------------------------------------------
// MXFP4 (e2m1 codes, one e8m0 scale per 32 elements of K) on the same skeleton: scaled 16x16x128
// f8f6f4 MFMAs, two per accumulator tile and K step (128 bytes of a row = 256 elements = 8 scale
// blocks of 16 bytes).  Lane (r, kg) of sub-step ks multiplies block 2 kg + ks of its row, which the loads have put into LDS slot 4 ks + kg.  (Which K positions
// a lane takes is free as long as A, B and the scales agree; but with the lane group in the LOW bits of the
// chunk number the fragment reads are free of LDS bank conflicts, with 2 kg + ks - the first version - every
// ds_read_b128 took 8 instead of 4 cycles: measured, SQ_LDS_BANK_CONFLICT = half of SQ_LDS_IDX_ACTIVE.)  The
// scales travel like the operands: 16 bytes per row (two K steps) per direct load into a two-slot LDS ring
// (row r at 16 r); from there the two scale bytes of a fragment and K step are fetched with one `ds_read_u16`.
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

// EPI: 0 = general epilogue, 3 / 4 = lean epilogue (gemm_epilogue16_lean) writing fp16 / bf16
// TAIL: K need not be a multiple of 1024 (of 32 still, the scale block): the main loop does the whole groups of four K
// steps, and what is left of each row (16 .. 496 bytes, the same for every tile) follows in K steps whose fragments and
// scale bytes every lane loads straight from global memory - zeros (and the scale 1) beyond K - into the fragment and
// scale registers that the pipeline has free at that point.
// BM = 192: tiles of 192 x 256 (a wave: 96 x 128, six A fragments, 48 of the tile's A rows and scale rows to fetch), for
// products whose 256 x 256 tiles fill the last round of CUs badly; lean epilogue, K steps in whole groups.
template <int EPI, bool TAIL = false, int BM = 256>
__device__ __forceinline__ void gemm_wave128_mxfp4_tiles(const GemmArgs& p, int tile, const int tile_step, LDS_PTR(char) const lds_raw) {
  static_assert(BM == 256 || ((BM == 192 || BM == 128) && !TAIL && (EPI == 3 || EPI == 4)), "192- and 128-row tiles: lean epilogue, no K tail");
#if MI355_DEVICE_PASS
  constexpr int BN = 256, ROWB = 128;
  constexpr int A_BYTES = BM * ROWB, STAGE = A_BYTES + BN * ROWB;  // 64 KiB (56 KiB)
  constexpr int SC_BASE = 2 * STAGE, SC_SLOT = (256 + BN) * 16;     // scale ring behind the two stages (A part: room for 256 rows)
  constexpr int MT = BM / 32, NT = 8, KS = 2, NM = MT * NT, NRD = MT + NT;
  constexpr int LA = BM / 32, NLOADS = LA + 8;                      // direct loads per wave and K step: A, then B
  constexpr int EVERY = NM / 16;                                    // MFMAs per load slot: 4 (64 MFMAs) or 3 (48)
  const unsigned lds0 = lds_addr((LDS_PTR(const void))lds_raw);

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int l16 = lane & 15, kg = lane >> 4;

  const int num_m = p.M / BM, num_n = p.N / BN;
  const int ntiles = num_m * num_n;
  int pm, pn;   // (the tiles tile, tile + tile_step, ... are computed as one stream of K steps)
  grouped_tile(xcd_remap(tile, ntiles), num_m, num_n, p.group_m, pm, pn);
  const int nk = TAIL ? p.k_bytes / (4 * ROWB) * 4 : p.k_bytes / ROWB;
  int nk_last = nk;   // the same number, but opaque: see mfma_retire
  asm volatile("" : "+s"(nk_last));

  // ---- operand loads, as in the 16-bit kernel
  // (a lane offset per load - row, chunk, and the instruction offset taken back out - and one scalar base per
  // operand that moves with the K step being fetched)
  const unsigned drow = lane >> 3, dslot = lane & 7;
  unsigned voffA[LA], voffB[8];
#pragma unroll
  for (int q = 0; q < 8; q++) {
    // (LDS slot s of a row takes the row's chunk 2 (s & 3) + (s >> 2): the fragment reads keep their conflict-free
    // slots 4 ks + kg and find the chunks 2 kg + ks there - the two scale blocks of a lane are then neighbours)
    const unsigned slot = dslot ^ (((q & 1) * 4 + (lane >> 4)) & 7);
    const unsigned chunk = 2 * (slot & 3) + (slot >> 2);
    if (q < LA) voffA[q] = (drow + 8 * q) * (unsigned)p.lda + chunk * 16 - (unsigned)((q - 4) * 1024);
    voffB[q] = (drow + 8 * q) * (unsigned)p.ldb + chunk * 16 - (unsigned)((q - 4) * 1024);
  }
  // scalar bases (operands and scales) of the tile the loads are fetching, two K steps ahead of the MFMAs
  const char* fA;   // operands: the K step being fetched
  const char* fB;
  const char* gSA;
  const char* gSB;
  // L2 touches two K steps ahead of the loads, as in the 16-bit kernel: the programs of an XCD's 8 x 4 patch of
  // tiles share out the lines of the panels they have in common
  constexpr bool PF = MI355_W128_PREFETCH;
  constexpr int PFD = MI355_W128_PREFETCH_DISTANCE;
  const char* pA = nullptr;
  const char* pB = nullptr;
  const unsigned voffPA = (lane % (BM / 16)) * (unsigned)p.lda, voffPB = (lane & 7) * (unsigned)p.ldb;
  const unsigned touch_lds = lds0 + SC_BASE + 2 * SC_SLOT + wave * 256;
  auto set_fill_tile = [&](int fm, int fn) {
    fA = p.A + ((int64_t)fm * BM + wave * (BM / 4)) * p.lda;
    fB = p.B + ((int64_t)fn * BN + wave * 64) * p.ldb;
    if constexpr (PF) {
      pA = p.A + ((int64_t)fm * BM + (fn & 3) * (BM / 4) + wave * (BM / 16)) * p.lda;
      pB = p.B + ((int64_t)fn * BN + (fm & 7) * 32 + wave * 8) * p.ldb;
    }
    gSA = (const char*)p.sA + ((int64_t)fm * BM + wave * (BM / 4)) * p.lds_a;
    gSB = (const char*)p.sB + ((int64_t)fn * BN + wave * 64) * p.lds_b;
  };
  set_fill_tile(pm, pn);
  auto load_of = [](int slot) constexpr { return slot < LA ? slot : 8 + slot - LA; };   // load slot -> j (A: 0 .. LA-1, B: 8 .. 15)
  auto issue = [&](auto J_, const char* srcA, const char* srcB, unsigned stage_base, auto SETTLE_) {
    constexpr int j = decltype(J_)::value, q = j & 7, ioff = (q - 4) * 1024;
    const unsigned dst = stage_base + (j < 8 ? wave * (LA * 1024) : A_BYTES + wave * 8192) + 4096;
    if constexpr (j < 8) async_copy16_sbase_off<ioff, q == 0, decltype(SETTLE_)::value>(srcA, voffA[q], dst);
    else async_copy16_sbase_off<ioff, q == 0, decltype(SETTLE_)::value>(srcB, voffB[q], dst);
  };
  // ---- scale loads: wave w fetches the 16 scale bytes (K steps 2 h, 2 h + 1) of its BM / 4 rows of A (192-row tiles: the
  // lanes beyond row 47 sit the load out) and of rows 64 w .. 64 w + 63 of B
  const unsigned voffSA = lane * (unsigned)p.lds_a, voffSB = lane * (unsigned)p.lds_b;
  auto issue_scales = [&](int h, auto SETTLE_) {   // pair h of K steps of the fill tile -> slot h & 1 (K steps come in fours, so
    const unsigned slot = lds0 + SC_BASE + (h & 1) * SC_SLOT;   // the slots alternate across tiles too)
    if (BM == 256 || lane < BM / 4) async_copy16_sbase<decltype(SETTLE_)::value>(gSA, voffSA + (unsigned)h * 16, slot + wave * (BM / 4) * 16);
    async_copy16_sbase<decltype(SETTLE_)::value>(gSB, voffSB + (unsigned)h * 16, slot + 256 * 16 + wave * 1024);
  };

  // ---- fragment reads: lane (l16, kg) of sub-step ks wants chunk 2 kg + ks of row l16 (+ 16 t)
  unsigned adrA[KS], adrB[KS];
  {
    const unsigned s = (l16 >> 1) & 7;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      const unsigned slot = ((4 * ks + kg) ^ s) * 16;
      adrA[ks] = lds0 + (wm * (BM / 2) + l16) * ROWB + slot;
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
  // scales: lane (r, kg) multiplies block 2 kg of its row in sub-step 0 and block 2 kg + 1 in sub-step 1: ONE 16-bit
  // read per fragment and K step fetches both (bytes 0 and 1 of the register, which the MFMA's compile-time selector
  // names: no shift), into the register set of the step's parity, read during the second half of the step before.
  const unsigned adrSA = lds0 + SC_BASE + (wm * (BM / 2) + l16) * 16 + 2 * kg;
  const unsigned adrSB = lds0 + SC_BASE + 256 * 16 + (wn * 128 + l16) * 16 + 2 * kg;
  int sa[2][MT], sb[2][NT];
  auto read_scale = [&](auto OP_, auto SET_, auto OFF_) {   // OFF: slot * SC_SLOT + (K step & 1) * 8
    constexpr int op = decltype(OP_)::value, set = decltype(SET_)::value, off = decltype(OFF_)::value;
    if constexpr (op < MT) sa[set][op] = lds_read_u16<off + op * 256>(adrSA);
    else sb[set][op - MT] = lds_read_u16<off + (op - MT) * 256>(adrSB);
  };
  auto pin_scales = [&](auto SET_) {
    constexpr int set = decltype(SET_)::value;
    static_for<MT>([&](auto T_) { lds_use(sa[set][decltype(T_)::value]); });
    static_for<NT>([&](auto T_) { lds_use(sb[set][decltype(T_)::value]); });
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
  issue_scales(0, std::true_type{});
  static_for<NLOADS>([&](auto L_) { issue(std::integral_constant<int, load_of(decltype(L_)::value)>{}, fA, fB, lds0, std::true_type{}); });
  static_for<NLOADS>([&](auto L_) { issue(std::integral_constant<int, load_of(decltype(L_)::value)>{}, fA + ROWB, fB + ROWB, lds0 + STAGE, std::true_type{}); });
  fA += 2 * ROWB;
  fB += 2 * ROWB;
  if constexpr (PF) {
    // the lines of K steps 2 and 3 (the loop's touches begin with step 2 + PFD); also the two youngest loads that
    // the loop's waits leave outstanding from the first step on
    const int k2 = min(2, nk - 1), k3 = min(3, nk - 1);
    touch_line_sbase<true, BM / 16>(pA + k2 * ROWB, voffPA, touch_lds);
    touch_line_sbase<false, 8>(pB + k2 * ROWB, voffPB, 0u);
    touch_line_sbase<false, BM / 16>(pA + k3 * ROWB, voffPA, 0u);
    touch_line_sbase<false, 8>(pB + k3 * ROWB, voffPB, 0u);
    pA += 2 * ROWB;
    pB += 2 * ROWB;
  }
  wait_vmcnt<NLOADS + (PF ? 4 : 0)>();
  block_barrier();
  static_for<NRD>([&](auto OP_) { read_one(OP_, I0{}, I0{}, f[0]); });
  static_for<NRD>([&](auto OP_) { read_scale(OP_, I0{}, I0{}); });
  lds_wait<0>();
  pin_scales(I0{});

  // K step U (0..3 within a group of four: stage U & 1, scale slot U >> 1)
  auto step = [&](auto U_, int fk) {   // fk: the K step (of the fill tile) that this step's loads fetch
    constexpr int U = decltype(U_)::value, P = U & 1, UN = (U + 1) & 3;
    using OffNext = std::integral_constant<int, (UN >> 1) * SC_SLOT + (UN & 1) * 8>;
    // sub-step 0 (blocks 2 kg); meanwhile the fragments of sub-step 1
    static_for<NM>([&](auto N_) {
      constexpr int n = decltype(N_)::value, i = n / NT, j = n % NT;
      mfma16_mxfp4<0>(f[0].b[j], f[0].a[i], acc[i][j], sb[P][j], sa[P][i]);
      if constexpr (n % 2 == 0 && n / 2 < NRD) read_one(std::integral_constant<int, n / 2>{}, std::integral_constant<int, P>{}, I1{}, f[1]);
      if constexpr (n % 2 == 1) __builtin_amdgcn_sched_barrier(0);
    });
    // sub-step 1 (blocks 2 kg + 1): meet, then read the next step's first fragments and scales and refill this stage
    lds_wait<0>();
    pin(f[1]);
    wait_vmcnt<PF ? 2 : 0>();   // (all but the two touches of the previous step, which are the youngest loads)
    block_barrier();
    static_for<NM>([&](auto N_) {
      constexpr int n = decltype(N_)::value, i = n / NT, j = n % NT;
      mfma16_mxfp4<1>(f[1].b[j], f[1].a[i], acc[i][j], sb[P][j], sa[P][i]);
      if constexpr (n % 2 == 0 && n / 2 < NRD) read_one(std::integral_constant<int, n / 2>{}, std::integral_constant<int, P ^ 1>{}, I0{}, f[0]);
      if constexpr (n % 2 == 1 && n / 2 < NRD) read_scale(std::integral_constant<int, n / 2>{}, std::integral_constant<int, P ^ 1>{}, OffNext{});
      if constexpr (n % EVERY == 1 && n / EVERY < NLOADS) issue(std::integral_constant<int, load_of(n / EVERY)>{}, fA, fB, lds0 + P * STAGE, std::false_type{});   // one per 64 (48) cycles
      // (the scales of the K steps fk, fk + 1 are requested in the even steps, into the slot that the pair
      // two steps back used: its last readers were the reads of that pair's second step, in its sub-step 0)
      // (after the last operand load: the eight loads of an operand share the M0 value that the first one sets)
      if constexpr (P == 0 && n == NM - 2) issue_scales(fk >> 1, std::false_type{});
      if constexpr (n % 2 == 1) __builtin_amdgcn_sched_barrier(0);
    });
    if constexpr (PF) {
      touch_line_sbase<true, BM / 16>(pA + (fk + PFD < nk ? PFD * ROWB : 0), voffPA, touch_lds);
      touch_line_sbase<false, 8>(pB + (fk + PFD < nk ? PFD * ROWB : 0), voffPB, 0u);
    }
    // everything requested above has landed before the registers are touched again
    lds_wait<0>();
    pin(f[0]);
    pin_scales(std::integral_constant<int, P ^ 1>{});
  };
  using I2 = std::integral_constant<int, 2>; using I3 = std::integral_constant<int, 3>;
  lds_wait<0>();
  pin(f[0]);
  // The fill cursor runs two K steps ahead of the MFMAs, across tile boundaries; behind the last tile it
  // wraps to that tile's first steps again (fetched into stages nobody reads any more), which keeps the
  // loop, the number of loads in flight and every wait uniform.
  int fk = 2, ftile = tile;
  auto advance = [&]() {
    fA += ROWB;
    fB += ROWB;
    if constexpr (PF) { pA += ROWB; pB += ROWB; }
    if (++fk == nk) {
      fk = 0;
      if (ftile + tile_step < ntiles) ftile += tile_step;
      int fm, fn;
      grouped_tile(xcd_remap(ftile, ntiles), num_m, num_n, p.group_m, fm, fn);
      set_fill_tile(fm, fn);
    }
  };
  while (true) {
    if constexpr (PF) wait_all();   // (once per tile: tells the compiler that its own loads have landed, see the 16-bit kernel)
    for (int kt = 0; kt < nk; kt += 4) {
      step(I0{}, fk); advance();
      step(I1{}, fk); advance();
      step(I2{}, fk); advance();
      step(I3{}, fk); advance();
      if (kt + 4 >= nk_last) mfma_retire();
    }
    if constexpr (TAIL) {
      // (free here: the fragment set 1 and the scale set 1 - the last step read the next tile's first fragments and
      // scales into the sets 0)
      const int k_main = nk * ROWB, tail = p.k_bytes - k_main;
      int tm = pm * BM + wm * 128, tn = pn * BN + wn * 128, tl = l16, tk = kg;
      asm volatile("" : "+s"(tm), "+s"(tn), "+v"(tl), "+v"(tk));   // (keeps this address arithmetic out of the K loop)
      // a scalar base per fragment and one 32-bit lane offset per operand (gemm_wave128_mxfp4_ok bounds them)
      const char* const tA = p.A + (int64_t)tm * p.lda + k_main;
      const char* const tB = p.B + (int64_t)tn * p.ldb + k_main;
      const uint8_t* const tSA = p.sA + (int64_t)tm * p.lds_a + k_main / 16;
      const uint8_t* const tSB = p.sB + (int64_t)tn * p.lds_b + k_main / 16;
      const unsigned offA = (unsigned)tl * (unsigned)p.lda + tk * 32, offB = (unsigned)tl * (unsigned)p.ldb + tk * 32;
      const unsigned offSA = (unsigned)tl * (unsigned)p.lds_a + tk * 2, offSB = (unsigned)tl * (unsigned)p.lds_b + tk * 2;
      for (int h = 0; h * ROWB < tail; h++) {
        // the blocks 2 tk (sub-step 0) and 2 tk + 1 (sub-step 1) of the step; their scales in bytes 0 and 1
        const bool ok0 = h * ROWB + tk * 32 < tail, ok1 = h * ROWB + tk * 32 + 16 < tail;
        auto scale = [&](const uint8_t* src, unsigned off) {
          int v0 = 127, v1 = 127;   // (2^0: multiplies zeros)
          if (ok0) v0 = src[h * 8 + (uint64_t)off];
          if (ok1) v1 = src[h * 8 + 1 + (uint64_t)off];
          return v0 | (v1 << 8);
        };
#pragma unroll
        for (int t = 0; t < MT; t++) sa[1][t] = scale(tSA + (int64_t)t * 16 * p.lds_a, offSA);
#pragma unroll
        for (int t = 0; t < NT; t++) sb[1][t] = scale(tSB + (int64_t)t * 16 * p.lds_b, offSB);
        static_for<KS>([&](auto KS_) {
          constexpr int ks = decltype(KS_)::value;
          const bool ok = ks == 0 ? ok0 : ok1;
          auto frag = [&](const char* src, unsigned off) {
            i32x4 v = {0, 0, 0, 0};
            if (ok) v = *(const i32x4*)(src + h * ROWB + ks * 16 + (uint64_t)off);
            return v;
          };
#pragma unroll
          for (int t = 0; t < MT; t++) f[1].a[t] = frag(tA + (int64_t)t * 16 * p.lda, offA);
#pragma unroll
          for (int t = 0; t < NT; t++) f[1].b[t] = frag(tB + (int64_t)t * 16 * p.ldb, offB);
          settle_pass(sa[1][0], sa[1][1], sa[1][2], sa[1][3], sa[1][4], sa[1][5], sa[1][6], sa[1][7],
                      sb[1][0], sb[1][1], sb[1][2], sb[1][3], sb[1][4], sb[1][5], sb[1][6], sb[1][7]);
          settle_tail(f[1].a[0], f[1].a[1], f[1].a[2], f[1].a[3], f[1].a[4], f[1].a[5], f[1].a[6], f[1].a[7],
                      f[1].b[0], f[1].b[1], f[1].b[2], f[1].b[3], f[1].b[4], f[1].b[5], f[1].b[6], f[1].b[7]);
          static_for<NM>([&](auto N_) {
            constexpr int n = decltype(N_)::value, i = n / NT, j = n % NT;
            mfma16_mxfp4<ks>(f[1].b[j], f[1].a[i], acc[i][j], sb[1][j], sa[1][i]);
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
    else gemm_epilogue16<MT, NT>(acc, p, em, en, el, ek);
    tile += tile_step;
    if (tile >= ntiles) break;
    grouped_tile(xcd_remap(tile, ntiles), num_m, num_n, p.group_m, pm, pn);
    zero_acc();
  }
  wait_vmcnt<0>();  // nothing may still be writing LDS when the workgroup ends
#endif
}

// Workgroup b computes the tiles b, b + gridDim.x, ... (the grid: wave128_grid).
template <int EPI, bool TAIL = false, int BM = 256>
__global__ __launch_bounds__(256, 1) void gemm_wave128_mxfp4_kernel(GemmArgs p) {
#if MI355_DEVICE_PASS
  extern __shared__ __attribute__((aligned(1024))) char lds_raw[];
  gemm_wave128_mxfp4_tiles<EPI, TAIL, BM>(p, blockIdx.x, gridDim.x, (LDS_PTR(char))lds_raw);
#endif
}

// Two tile heights in one launch, as for the 16-bit and fp8 products: the first `rows256` rows of C on tiles of 256 x 256,
// the rows below (their operand and scale rows) on tiles of 192 x 256 dealt from the other end of the grid.
template <int EPI>
__global__ __launch_bounds__(256, 1) void gemm_wave128_mxfp4_mixed_kernel(GemmArgs p, int rows256) {
#if MI355_DEVICE_PASS
  extern __shared__ __attribute__((aligned(1024))) char lds_raw[];
  const int G = gridDim.x, nn = p.N / 256;
  {
    GemmArgs q = p;
    q.M = rows256;
    if ((int)blockIdx.x < (rows256 / 256) * nn) gemm_wave128_mxfp4_tiles<EPI, false, 256>(q, blockIdx.x, G, (LDS_PTR(char))lds_raw);
  }
  block_barrier();   // (the stages are laid out differently from here on; every wave has waited for its own loads)
  {
    GemmArgs q = p;
    q.A = p.A + (int64_t)rows256 * p.lda;
    q.sA = p.sA + (int64_t)rows256 * p.lds_a;
    q.C = p.C + (int64_t)rows256 * p.ldc * 2;
    q.M = p.M - rows256;
    const int j = G - 1 - (int)blockIdx.x;
    if (j < (q.M / 192) * nn) gemm_wave128_mxfp4_tiles<EPI, false, 192>(q, j, G, (LDS_PTR(char))lds_raw);
  }
#endif
}

template <int EPI>
static int launch_wave128_mxfp4_mixed(const GemmArgs& p, int rows256, hipStream_t stream) {
  constexpr int smem = 2 * (256 + 256) * 128 + 2 * 512 * 16 + 1024;
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)gemm_wave128_mxfp4_mixed_kernel<EPI>, hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) return (int)e;
    attr_set = true;
  }
  const int grid = p.num_programs > 0 ? p.num_programs : 256;
  gemm_wave128_mxfp4_mixed_kernel<EPI><<<dim3(grid), dim3(256), smem, stream>>>(p, rows256);
  return (int)hipGetLastError();
}

// fmt: 0 = MXFP4, else MXFP8 (gemm_wave128_mx_mixed_ok: lean epilogue)
int gemm_wave128_mx_mixed_launch(const GemmArgs& p, int fmt, int rows256, hipStream_t stream) {
  const int lean = lean_epilogue_type(p);
  if (fmt == 0) return lean == 1 ? launch_wave128_mxfp4_mixed<3>(p, rows256, stream) : launch_wave128_mxfp4_mixed<4>(p, rows256, stream);
  return lean == 1 ? launch_wave128_mxfp8_mixed<3>(p, rows256, stream) : launch_wave128_mxfp8_mixed<4>(p, rows256, stream);
}

// the first `rows256` rows on 256-row tiles and the rest on 192-row tiles, under the conditions of the 192-row tiles
bool gemm_wave128_mx_mixed_ok(const GemmArgs& p, int group_bytes, int rows256) {
  if (!(rows256 > 0 && rows256 < p.M && rows256 % 256 == 0 && (p.M - rows256) % 192 == 0)) return false;
  GemmArgs q = p;
  q.M = 768;   // (a multiple of both tile heights: the other conditions of gemm_wave128_mx_192_ok)
  return gemm_wave128_mx_192_ok(q, group_bytes, 192);
}

// the block-scaled forms on tiles of 192 x 256: M a multiple of 192, whole groups of K steps (`group_bytes` of a row: 512
// for MXFP4, 1024 for MXFP8), a 16-bit C through the lean epilogue
bool gemm_wave128_mx_192_ok(const GemmArgs& p, int group_bytes, int tile_m) {
  return p.M % tile_m == 0 && p.N % 256 == 0 && p.k_bytes % group_bytes == 0 && p.k_bytes >= group_bytes && lean_epilogue_type(p) != 0 &&
         p.lda * 8 + p.k_bytes < (1ll << 31) && p.ldb * 8 + p.k_bytes < (1ll << 31) &&
         p.lds_a % 16 == 0 && p.lds_b % 16 == 0 && ((uintptr_t)p.sA | (uintptr_t)p.sB) % 16 == 0 &&
         p.lds_a * 64 + p.k_bytes / 16 < (1ll << 31) && p.lds_b * 64 + p.k_bytes / 16 < (1ll << 31);
}

bool gemm_wave128_mxfp4_ok(const GemmArgs& p) {
  // whole tiles, at least one group of four K steps (K >= 1024 elements; what is left behind the last group: the TAIL
  // form), scale rows that a 16-byte load can fetch
  return p.M % 256 == 0 && p.N % 256 == 0 && p.k_bytes % 16 == 0 && p.k_bytes >= 512 &&
         p.lda * 8 + p.k_bytes < (1ll << 31) && p.ldb * 8 + p.k_bytes < (1ll << 31) &&
         p.lds_a % 16 == 0 && p.lds_b % 16 == 0 && ((uintptr_t)p.sA | (uintptr_t)p.sB) % 16 == 0 &&
         p.lds_a * 64 + p.k_bytes / 16 < (1ll << 31) && p.lds_b * 64 + p.k_bytes / 16 < (1ll << 31);
}

template <int EPI, bool TAIL = false, int BM = 256>
static int launch_wave128_mxfp4(const GemmArgs& p, hipStream_t stream) {
  constexpr int smem = 2 * (BM + 256) * 128 + 2 * 512 * 16 + 1024;   // (stages, scale ring and the 1 KiB that the L2 touches land in)
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)gemm_wave128_mxfp4_kernel<EPI, TAIL, BM>, hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) return (int)e;
    attr_set = true;
  }
  const int tiles = (p.M / BM) * (p.N / 256);
  const int grid = wave128_grid(tiles, p.num_programs);
  gemm_wave128_mxfp4_kernel<EPI, TAIL, BM><<<dim3(grid), dim3(256), smem, stream>>>(p);
  return (int)hipGetLastError();
}

int gemm_wave128_mxfp4_launch(const GemmArgs& p, hipStream_t stream) {
  const int lean = lean_epilogue_type(p);
  if (p.tile_m == 192)   // (gemm_wave128_mx_192_ok: lean epilogue, whole groups of K steps)
    return lean == 1 ? launch_wave128_mxfp4<3, false, 192>(p, stream) : launch_wave128_mxfp4<4, false, 192>(p, stream);
  if (p.tile_m == 128)
    return lean == 1 ? launch_wave128_mxfp4<3, false, 128>(p, stream) : launch_wave128_mxfp4<4, false, 128>(p, stream);
  if (p.k_bytes % 512 != 0)
    return lean == 1 ? launch_wave128_mxfp4<3, true>(p, stream) : lean == 2 ? launch_wave128_mxfp4<4, true>(p, stream) : launch_wave128_mxfp4<0, true>(p, stream);
  return lean == 1 ? launch_wave128_mxfp4<3>(p, stream) : lean == 2 ? launch_wave128_mxfp4<4>(p, stream) : launch_wave128_mxfp4<0>(p, stream);
}

}  // namespace mi355

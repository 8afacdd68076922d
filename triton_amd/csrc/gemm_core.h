// Tiled MFMA GEMM core for gfx950, shared by the fp16/bf16, fp8 and block-scaled MX kernels:
//   C[M,N] = act(alpha * A[M,K] @ B[K,N]), fp32 accumulate.
//
// The device-side counterpart of the reference `matmul_kernel`
// (python/tutorials/03-matrix-multiplication.py:241-316): one workgroup per BM x BN tile of C,
// grouped tile order (:265-273), K loop (:294-303), epilogue activation and cast (:304-316).
// Built MI355X-first instead of translated:
//   * a K step is RBK = 64 BYTES of every operand row (32 fp16/bf16, 64 fp8, 128 fp4 elements);
//     tiles go global -> LDS with direct 16-byte loads into a ring of NS LDS stages (no register
//     staging).  Loads run NS-1 steps ahead of the MFMAs: an L2 round trip under load is longer
//     than one step, so a two-stage ring stalls every step on its own prefetch;
//   * one barrier per step, entered after waiting only for the loads of the step about to be
//     multiplied (the younger ones stay in flight);
//   * LDS rows are XOR-swizzled for the 64-bank LDS so that ds_read_b128 / ds_read_b64_tr_b16
//     are conflict free;
//   * a row-major 16-bit or fp8 B[K,N] is transposed on the fly by the LDS transpose reads; a K-major B
//     (the `b.T` view the reference passes for fp8, :378-382) uses plain 128-bit reads;
//   * 32x32 MFMA tiles with the operands swapped, so every lane owns 4 consecutive columns of
//     one C row and stores them with one instruction;
//   * workgroup ids are remapped per XCD before the grouped ordering.
//
// `Cfg` describes one element family:
//   kSteps            MFMA sub-steps per 64-byte K step
//   kChunks           16-byte LDS chunks one lane feeds into one MFMA operand (1 or 2)
//   chunk(ks, g, c)   which 16-byte chunk (0..3) of the row lane-group g reads for sub-step ks
//   kRowMajorB        whether a transpose-read path for a row-major B exists (16-bit: every kernel form; fp8: the
//                     one-barrier-per-step form)
//   kElemBytes        bytes per element of a row-major B (2 or 1; unused without kRowMajorB)
//   kScaled           block-scaled: per-row e8m0 scales ride along (MX)
//   Operand           register type of one MFMA operand
//   mma<ks>(...)      the MFMA itself
#pragma once
#include "common.h"
#include "launch.h"

namespace mi355 {

constexpr int RBK = 64;          // bytes of one operand row per K step
constexpr int CPR = RBK / 16;    // 16-byte chunks per row of a K-major LDS tile

// K-major LDS tile: rows of RBK bytes, four rows per 256-byte bank sweep.  A ds_read_b128 is
// served 16 lanes at a time; 16 consecutive rows reading the same logical chunk must hit 16
// different 16-byte slots of the sweep.  The slot is (row & 3) * 4 + chunk, so the chunk index
// is XORed with bits 2..3 of the row.
__device__ __forceinline__ int kswz(int row) { return (row >> 2) & (CPR - 1); }
__device__ __forceinline__ int kmajor_off(int row, int chunk) { return row * RBK + (((chunk ^ kswz(row))) << 4); }

// Direct global -> LDS copy of a K-major [ROWS x RBK] tile.  One wave instruction moves
// 64 x 16 B = 16 rows; the LDS side of such a load is linear in the lane id, so the swizzle is
// applied to the SOURCE chunk each lane fetches.
template <int ROWS, int NW>
struct TileCopyK {
  static constexpr int kRowsPerInst = 1024 / RBK;
  static constexpr int kIters = ROWS / kRowsPerInst / NW;
  static_assert(ROWS % (kRowsPerInst * NW) == 0 && kIters >= 1, "tile rows must split evenly over the waves");
  __device__ static int row(int wave, int lane, int i) { return (i * NW + wave) * kRowsPerInst + lane / CPR; }
  __device__ static int chunk(int lane, int r) { return (lane % CPR) ^ kswz(r); }  // logical chunk fetched
};

// Row-major [RBK/EB x BN] tile of B with elements of EB bytes (rows are k, BN*EB bytes each).
// 16-bit: a transpose read is served 32 lanes at a time: two 16-lane groups that address the same 4
// consecutive k rows and two neighbouring 32-byte groups of columns.  The 32-byte group index is XORed
// with 2 * (k & 3), which spreads those 4 rows x 64 bytes over all banks.
// 8-bit: a transpose read (ds_read_b64_tr_b8: within 16 lanes, lane 2 r + h addresses the 8 bytes of columns
// 8 h .. 8 h + 7 of row r; lane j receives column j of the 8 rows) covers, per 32 lanes, 8 consecutive k rows of
// two neighbouring 16-byte chunks.  The chunk index is XORed with twice the row's number among the rows that
// share a 16-byte bank column (every row when a row is a whole 256-byte bank sweep, every second when it is half
// of one), which puts those 16 pieces on 16 different bank groups.
template <int BN, int NW, int EB = 2>
struct TileCopyKN {
  static constexpr int kRows = RBK / EB;
  static constexpr int kChunksPerRow = BN * EB / 16;       // 16-byte chunks per k row
  static constexpr int kRowsPerInst = 64 / kChunksPerRow;  // k rows moved by one wave instruction
  static constexpr int kIters = kRows / kRowsPerInst / NW;
  static constexpr int kRowsPerSweep = 256 / (BN * EB) > 0 ? 256 / (BN * EB) : 1;
  static_assert(kRowsPerInst >= 1 && kIters >= 1, "tile too small for this wave count");
  static_assert(EB == 2 || ((7 / kRowsPerSweep) << 1) < kChunksPerRow, "the 8-bit swizzle needs that many chunks per row");
  __device__ static int row(int wave, int lane, int i) { return (i * NW + wave) * kRowsPerInst + lane / kChunksPerRow; }
  __device__ static int swz8(int r) { return ((r & 7) / kRowsPerSweep) << 1; }
  __device__ static int col16(int lane, int r) {  // logical 16-byte chunk this lane fetches
    int pc16 = lane % kChunksPerRow;
    if constexpr (EB == 1) {
      return pc16 ^ swz8(r);
    } else {
      int lc32 = (pc16 >> 1) ^ ((r & 3) << 1);
      return lc32 * 2 + (pc16 & 1);
    }
  }
};

// Epilogue shared by the GEMM kernels: alpha, activation, cast, store.  With the operands
// swapped (D[n][m]) lane l owns C row `mrow0 + 32 i + l%32` and, per register group rg of tile
// (i, j), the four consecutive columns `ncol0 + 32 j + 8 rg + 4 (l/32) ..`.
template <int MT, int NT>
__device__ __forceinline__ void gemm_epilogue(f32x16 (&acc)[MT][NT], const GemmArgs& p, int mrow0, int ncol0, int l32, int g) {
  // epilogue: lane owns row m = .. + l32 and, per register group rg, columns n .. n+3.
  // The tile loops are compile-time recursions, not `#pragma unroll`: with a body this size the
  // unroller may give up, and a runtime index into `acc` would move the accumulators to scratch memory.
  float alpha = 1.f;
  if (p.a_scale) alpha *= *p.a_scale;
  if (p.b_scale) alpha *= *p.b_scale;
  // The common case first, as a short path of its own: the wave's tile lies inside C, C is fp16 / bf16 with unit
  // column stride and aligned rows, no activation, no addend.  The general path below decides all of that per
  // group of four values inside the unrolled tiles - tens of KiB of code that the instruction cache has to
  // fetch at the end of every tile (the four-wave kernels, whose epilogue is the same in larger, gained 4-15 %
  // from a lean instantiation; here the choice is a branch, uniform over the workgroup).
  if (p.lean_ok && !p.aux && p.activation == 0 && p.scn == 1 && p.c_vec_ok && p.ldc % 8 == 0 && (p.out_dtype == 0 || p.out_dtype == 1) &&
      mrow0 + MT * 32 <= p.M && ncol0 + NT * 32 <= p.N) {
    // (Rows of 16-byte alignment.)  Register groups 2 a and 2 a + 1 are exchanged between the two lanes of a row
    // (v_permlane32_swap) - lane l32 then holds the 8 consecutive columns 16 a .. 16 a + 7 of the tile, lane
    // l32 + 32 the next 8 - and a lane stores 16 bytes instead of two pieces of 8: half the requests to the memory
    // pipeline, which takes one per piece (see gemm_epilogue16_lean of the four-wave kernels).
    auto lean16 = [&](auto* c0) {
      using OutT = std::remove_pointer_t<decltype(c0)>;
      typedef OutT Out2 __attribute__((ext_vector_type(2)));
      static_for<MT>([&](auto I_) {
        constexpr int i = decltype(I_)::value;
        OutT* row = c0 + (int64_t)(mrow0 + i * 32 + l32) * p.ldc + ncol0 + g * 8;
        static_for<NT>([&](auto J_) {
          constexpr int j = decltype(J_)::value;
#pragma unroll
          for (int a = 0; a < 2; a++) {
            int x0 = __builtin_bit_cast(int, Out2{(OutT)(acc[i][j][a * 8] * alpha), (OutT)(acc[i][j][a * 8 + 1] * alpha)});
            int x1 = __builtin_bit_cast(int, Out2{(OutT)(acc[i][j][a * 8 + 2] * alpha), (OutT)(acc[i][j][a * 8 + 3] * alpha)});
            int y0 = __builtin_bit_cast(int, Out2{(OutT)(acc[i][j][a * 8 + 4] * alpha), (OutT)(acc[i][j][a * 8 + 5] * alpha)});
            int y1 = __builtin_bit_cast(int, Out2{(OutT)(acc[i][j][a * 8 + 6] * alpha), (OutT)(acc[i][j][a * 8 + 7] * alpha)});
            swap32_regs(x0, y0);
            swap32_regs(x1, y1);
            *(i32x4*)(row + j * 32 + a * 16) = i32x4{x0, x1, y0, y1};
          }
        });
      });
    };
    if (p.out_dtype == 1) lean16((__bf16*)p.C); else lean16((_Float16*)p.C);
    return;
  }
  const bool leaky = p.activation == 1;
  const bool vec_ok = p.c_vec_ok;
  const bool has_aux = p.aux != nullptr;
  static_for<MT>([&](auto I_) {
    constexpr int i = decltype(I_)::value;
    const int m = mrow0 + i * 32 + l32;
    if (m < p.M) {
      static_for<NT>([&](auto J_) {
        constexpr int j = decltype(J_)::value;
        static_for<4>([&](auto RG_) {
          constexpr int rg = decltype(RG_)::value;
          const int n = ncol0 + j * 32 + rg * 8 + g * 4;
          float v[4];
#pragma unroll
          for (int e = 0; e < 4; e++) v[e] = acc[i][j][rg * 4 + e] * alpha;
          if (has_aux) {
#pragma unroll
            for (int e = 0; e < 4; e++)
              if (n + e < p.N) v[e] += load_aux(p.aux, (int64_t)m * p.aux_sm + (int64_t)(n + e) * p.aux_sn, p.aux_dtype);
          }
          if (leaky) {
#pragma unroll
            for (int e = 0; e < 4; e++) v[e] = v[e] >= 0.f ? v[e] : 0.01f * v[e];
          }
          if (p.out_dtype == 2 || p.out_dtype == 3) {
            const int count = p.N - n < 4 ? p.N - n : 4;
            if (count > 0) store4_fp8(p.C, (int64_t)m * p.ldc + (int64_t)n * p.scn, p.scn, p.out_dtype, v, vec_ok, count);
          } else if (p.out_dtype == 4) {
            float* c = (float*)p.C + (int64_t)m * p.ldc + (int64_t)n * p.scn;
            if (vec_ok && n + 3 < p.N) {
              *(f32x4*)c = f32x4{v[0], v[1], v[2], v[3]};
            } else {
#pragma unroll
              for (int e = 0; e < 4; e++) if (n + e < p.N) c[e * p.scn] = v[e];
            }
          } else if (p.out_dtype == 1) {
            __bf16* c = (__bf16*)p.C + (int64_t)m * p.ldc + (int64_t)n * p.scn;
            if (vec_ok && n + 3 < p.N) {
              *(bf16x4*)c = bf16x4{(__bf16)v[0], (__bf16)v[1], (__bf16)v[2], (__bf16)v[3]};
            } else {
#pragma unroll
              for (int e = 0; e < 4; e++) if (n + e < p.N) c[e * p.scn] = (__bf16)v[e];
            }
          } else {
            _Float16* c = (_Float16*)p.C + (int64_t)m * p.ldc + (int64_t)n * p.scn;
            if (vec_ok && n + 3 < p.N) {
              *(f16x4*)c = f16x4{(_Float16)v[0], (_Float16)v[1], (_Float16)v[2], (_Float16)v[3]};
            } else {
#pragma unroll
              for (int e = 0; e < 4; e++) if (n + e < p.N) c[e * p.scn] = (_Float16)v[e];
            }
          }
        });
      });
    }
  });
}

// One BM x BN tile of C (tile row pm, tile column pn) with a ring of NS LDS stages at `lds`
// (NS * (BM + BN) * RBK bytes).  Shared by the one-tile-per-workgroup kernel below and by the
// grouped kernel, whose workgroups walk the tiles of several problems.
template <typename Cfg, int BM, int BN, int WM, int WN, bool B_KMAJOR, int NS>
__device__ __forceinline__ void gemm_tile_body(const GemmArgs& p, const int pm, const int pn, LDS_PTR(char) const lds) {
  using Operand = typename Cfg::Operand;
  constexpr int NW = WM * WN, TM = BM / WM, TN = BN / WN, MT = TM / 32, NT = TN / 32;
  constexpr int A_BYTES = BM * RBK, B_BYTES = BN * RBK, STAGE = A_BYTES + B_BYTES;
  constexpr int KS = Cfg::kSteps, NC = Cfg::kChunks;
  static_assert(B_KMAJOR || Cfg::kRowMajorB, "row-major B needs a transpose read");
  constexpr int EB = Cfg::kElemBytes == 1 ? 1 : 2;   // element size of a row-major B (16-bit or fp8)
  using CopyA = TileCopyK<BM, NW>;
  using CopyBk = TileCopyK<BN, NW>;
  using CopyBn = TileCopyKN<BN, NW, EB>;
  constexpr int ITA = CopyA::kIters;
  constexpr int ITB = B_KMAJOR ? CopyBk::kIters : CopyBn::kIters;
  constexpr int KROWS = RBK / EB;  // k rows of a row-major B tile

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WN, wn = wave % WN;
  const int m0 = pm * BM, n0 = pn * BN;

  // per-lane global source pointers of the k = 0 tile; rows past the matrix edge are clamped
  // onto the last valid row (their products are never stored)
  const char* srcA[ITA];
  const char* srcB[ITB];
#pragma unroll
  for (int i = 0; i < ITA; i++) {
    int r = CopyA::row(wave, lane, i);
    int gr = min(m0 + r, p.M - 1);
    srcA[i] = p.A + (int64_t)gr * p.lda + CopyA::chunk(lane, r) * 16;
  }
#pragma unroll
  for (int i = 0; i < ITB; i++) {
    if constexpr (B_KMAJOR) {
      int r = CopyBk::row(wave, lane, i);
      int gr = min(n0 + r, p.N - 1);
      srcB[i] = p.B + (int64_t)gr * p.ldb + CopyBk::chunk(lane, r) * 16;
    } else {
      int r = CopyBn::row(wave, lane, i);
      int nb = n0 * EB + CopyBn::col16(lane, r) * 16;   // byte column of the chunk
      // (clamp whole chunks; the last chunk of a row may reach beyond N into the row's padding: the C ABI takes a
      // row-major B only with a pitch that covers N rounded up to whole chunks)
      const int nbytes = (p.N * EB + 15) / 16 * 16;
      nb = nb < nbytes ? nb : nbytes - 16;
      srcB[i] = p.B + (int64_t)r * p.ldb + nb;
    }
  }
  const int64_t stepA = RBK, stepB = B_KMAJOR ? (int64_t)RBK : KROWS * p.ldb;

  auto issue_tile = [&](int kt, LDS_PTR(char) a) {
    LDS_PTR(char) b = a + A_BYTES;
#pragma unroll
    for (int i = 0; i < ITA; i++) async_copy16(srcA[i] + kt * stepA, (LDS_PTR(void))(a + (i * NW + wave) * 1024));
#pragma unroll
    for (int i = 0; i < ITB; i++) async_copy16(srcB[i] + kt * stepB, (LDS_PTR(void))(b + (i * NW + wave) * 1024));
  };
  // Last, partial K tile: chunks past K are written as zeros (the reference masks them to 0,
  // python/tutorials/03-matrix-multiplication.py:297-298); goes through registers.
  auto guarded_tile = [&](int kt, LDS_PTR(char) a) {
    LDS_PTR(char) b = a + A_BYTES;
    const int kbase = kt * RBK;  // bytes along K
#pragma unroll
    for (int i = 0; i < ITA; i++) {
      int r = CopyA::row(wave, lane, i);
      i32x4 v = {0, 0, 0, 0};
      if (kbase + CopyA::chunk(lane, r) * 16 < p.k_bytes) v = *(const i32x4*)(srcA[i] + kt * stepA);
      *(LDS_PTR(i32x4))(a + (i * NW + wave) * 1024 + lane * 16) = v;
    }
#pragma unroll
    for (int i = 0; i < ITB; i++) {
      bool ok;
      if constexpr (B_KMAJOR) {
        int r = CopyBk::row(wave, lane, i);
        ok = kbase + CopyBk::chunk(lane, r) * 16 < p.k_bytes;
      } else {
        ok = kt * KROWS + CopyBn::row(wave, lane, i) < p.K;
      }
      i32x4 v = {0, 0, 0, 0};
      if (ok) v = *(const i32x4*)(srcB[i] + kt * stepB);
      *(LDS_PTR(i32x4))(b + (i * NW + wave) * 1024 + lane * 16) = v;
    }
  };

  f32x16 acc[MT][NT];
#pragma unroll
  for (int i = 0; i < MT; i++)
#pragma unroll
    for (int j = 0; j < NT; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

  // Per-lane LDS byte offsets of the MFMA operands inside one stage.
  //   K-major operand (A always, B when B_KMAJOR): lane reads row (l%32) and the 16-byte
  //   chunk(s) Cfg::chunk(ks, l/32, c), swizzled; 32-row sub-tiles add t * 32 * RBK.
  //   Row-major 16-bit B: transpose read, lane i of a 16-lane group q addresses k row
  //   16*ks + 8*(q/2) + i/4 (+4 for the second half) and 32-byte group (n/16) ^ 2*(k & 3).
  //   Row-major fp8 B: four transpose reads of 8 k rows each - rows 16 (q/2) + {0, 8, 32, 40} + i/2, the K positions
  //   of the two chunks (q/2, 2 + q/2) that the A operand of the same lane group holds - of the 16-byte chunk
  //   (n/16) ^ swz8(k), half i & 1; k & 7 and with it the swizzle are the same for all four.
  const int l32 = lane & 31, g = lane >> 5;
  const int i16 = lane & 15, q = lane >> 4;
  unsigned offA[KS][NC], offB[KS][NC];
#pragma unroll
  for (int ks = 0; ks < KS; ks++)
#pragma unroll
    for (int c = 0; c < NC; c++) {
      offA[ks][c] = kmajor_off(wm * TM + l32, Cfg::chunk(ks, g, c));
      offB[ks][c] = A_BYTES + kmajor_off(wn * TN + l32, Cfg::chunk(ks, g, c));
    }
  unsigned offBn[NT];
  if constexpr (EB == 1) {
    int k = (q >> 1) * 16 + (i16 >> 1);
#pragma unroll
    for (int t = 0; t < NT; t++) {
      int c16 = (wn * TN + t * 32) / 16 + (q & 1);
      offBn[t] = A_BYTES + k * BN + ((c16 ^ CopyBn::swz8(k)) << 4) + (i16 & 1) * 8;
    }
  } else {
    // k row without the ks / +4 terms; (k & 3) is the same for every ks and both halves
    int k = (q >> 1) * 8 + (i16 >> 2);
#pragma unroll
    for (int t = 0; t < NT; t++) {
      int c32 = (wn * TN + t * 32) / 16 + (q & 1);
      offBn[t] = A_BYTES + k * (BN * 2) + ((c32 ^ ((k & 3) << 1)) << 5) + (i16 & 3) * 8;
    }
  }

  struct Frags { Operand a[MT]; Operand b[NT]; };
  auto read_operand = [&](unsigned base, const unsigned (&off)[NC], auto IMM) -> Operand {
    constexpr int imm = decltype(IMM)::value;
    if constexpr (NC == 1) {
      return __builtin_bit_cast(Operand, lds_read_b128<imm>(base + off[0]));
    } else {
      i32x4 lo = lds_read_b128<imm>(base + off[0]);
      i32x4 hi = lds_read_b128<imm>(base + off[1]);
      i32x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
      return __builtin_bit_cast(Operand, both);
    }
  };
  auto read_frags = [&](unsigned base, auto KS_, Frags& f) {
    constexpr int ks = decltype(KS_)::value;
    static_for<MT>([&](auto T_) {
      constexpr int t = decltype(T_)::value;
      f.a[t] = read_operand(base, offA[ks], std::integral_constant<int, t * 32 * RBK>{});
    });
    static_for<NT>([&](auto T_) {
      constexpr int t = decltype(T_)::value;
      if constexpr (B_KMAJOR) {
        f.b[t] = read_operand(base, offB[ks], std::integral_constant<int, t * 32 * RBK>{});
      } else if constexpr (EB == 1) {
        static_assert(KS == 1 && NC == 2, "the fp8 transpose read feeds one 64-byte sub-step");
        i32x2 r0 = lds_read_tr8_b64<0>(base + offBn[t]);
        i32x2 r1 = lds_read_tr8_b64<8 * BN>(base + offBn[t]);
        i32x2 r2 = lds_read_tr8_b64<32 * BN>(base + offBn[t]);
        i32x2 r3 = lds_read_tr8_b64<40 * BN>(base + offBn[t]);
        i32x4 lo = __builtin_shufflevector(r0, r1, 0, 1, 2, 3);
        i32x4 hi = __builtin_shufflevector(r2, r3, 0, 1, 2, 3);
        i32x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        f.b[t] = __builtin_bit_cast(Operand, both);
      } else {
        constexpr int imm = ks * 16 * BN * 2;
        i32x2 lo = lds_read_tr16_b64<imm>(base + offBn[t]);
        i32x2 hi = lds_read_tr16_b64<imm + 4 * BN * 2>(base + offBn[t]);
        i32x4 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3);
        f.b[t] = __builtin_bit_cast(Operand, both);
      }
    });
  };
  constexpr int kReadsPerStep = MT * NC + NT * (B_KMAJOR ? NC : (EB == 1 ? 4 : 2));
  auto use_frags = [&](Frags& f) {
#pragma unroll
    for (int t = 0; t < MT; t++) lds_use(f.a[t]);
#pragma unroll
    for (int t = 0; t < NT; t++) lds_use(f.b[t]);
  };

  // block scales of the K step being multiplied and of the next one: one dword per 32-row
  // sub-tile and lane, already shifted so that byte `ks` is the scale of sub-step ks
  int sa[MT], sb[NT], sa_next[MT], sb_next[NT];
  auto load_scales = [&](int kt, int (&da)[MT], int (&db)[NT]) {
    if constexpr (Cfg::kScaled) {
#pragma unroll
      for (int t = 0; t < MT; t++) {
        int r = min(m0 + wm * TM + t * 32 + l32, p.M - 1);
        da[t] = Cfg::load_scale(p.sA + (int64_t)r * p.lds_a, kt, g);
      }
#pragma unroll
      for (int t = 0; t < NT; t++) {
        int r = min(n0 + wn * TN + t * 32 + l32, p.N - 1);
        db[t] = Cfg::load_scale(p.sB + (int64_t)r * p.lds_b, kt, g);
      }
    }
  };
  auto rotate_scales = [&]() {
    if constexpr (Cfg::kScaled) {
#pragma unroll
      for (int t = 0; t < MT; t++) sa[t] = sa_next[t];
#pragma unroll
      for (int t = 0; t < NT; t++) sb[t] = sb_next[t];
    }
  };

  auto mma = [&](const Frags& f, auto KS_) {
    constexpr int ks = decltype(KS_)::value;
#pragma unroll
    for (int i = 0; i < MT; i++)
#pragma unroll
      for (int j = 0; j < NT; j++) {
        // operands swapped: the instruction computes D[n][m]
        if constexpr (Cfg::kScaled) acc[i][j] = Cfg::template mma<ks>(f.b[j], f.a[i], acc[i][j], sb[j], sa[i]);
        else acc[i][j] = Cfg::template mma<ks>(f.b[j], f.a[i], acc[i][j], 0, 0);
      }
  };

  // One K step.  When the registers allow it, the operands of sub-step ks+1 are requested
  // before the MFMAs of sub-step ks; otherwise the second wave on the SIMD has to cover the LDS
  // latency.
  constexpr int kOperandRegs = (MT + NT) * NC * 4;
  constexpr bool kPrefetch = KS > 1 && 2 * kOperandRegs + MT * NT * 16 + (Cfg::kScaled ? 2 * (MT + NT) : 0) <= 184 * (512 / (NW * 64));
  auto compute_tile = [&](LDS_PTR(char) stage) {
    const unsigned base = lds_addr(stage);
    if constexpr (kPrefetch) {
      Frags f[2];
      read_frags(base, std::integral_constant<int, 0>{}, f[0]);
      static_for<KS>([&](auto KS_) {
        constexpr int ks = decltype(KS_)::value;
        if constexpr (ks + 1 < KS) {
          read_frags(base, std::integral_constant<int, ks + 1>{}, f[(ks + 1) & 1]);
          lds_wait<kReadsPerStep>();
        } else {
          lds_wait<0>();
        }
        use_frags(f[ks & 1]);
        mma(f[ks & 1], KS_);
      });
    } else {
      static_for<KS>([&](auto KS_) {
        Frags f;
        read_frags(base, KS_, f);
        lds_wait<0>();
        use_frags(f);
        mma(f, KS_);
      });
    }
  };

  // ---- K loop: loads run NS-1 steps ahead.  Step kt:  wait for the loads of tile kt only,
  //      barrier (every wave's part of tile kt is in LDS, and every wave has finished reading
  //      tile kt-1), refill the stage tile kt-1 occupied with tile kt+NS-1, multiply tile kt.
  const int nfull = p.k_bytes / RBK;
  constexpr int kLoadsPerTile = ITA + ITB;
  constexpr int kScaleLoads = Cfg::kScaled ? MT + NT : 0;
#pragma unroll
  for (int s = 0; s < NS - 1; s++)
    if (s < nfull) issue_tile(s, lds + s * STAGE);
  if (nfull > 0) load_scales(0, sa, sb);
  int stage = 0, fill = NS - 1;  // stage of tile kt, stage to refill
  for (int kt = 0; kt < nfull; kt++) {
    // Younger than the loads of tile kt are, in steady state, NS-2 whole steps (their tile
    // loads and the scale loads each of them issued) plus the scale loads of the step that issued
    // tile kt.  The prologue and the last steps issue fewer: they wait for everything.
    constexpr int kYounger = (NS - 2) * (kLoadsPerTile + kScaleLoads) + kScaleLoads;
    const bool steady = kt + NS - 2 < nfull && (!Cfg::kScaled || kt >= NS - 1);
    if (steady) wait_vmcnt<kYounger>(); else wait_vmcnt<0>();
    block_barrier();
    if (kt + NS - 1 < nfull) issue_tile(kt + NS - 1, lds + fill * STAGE);
    if (kt + 1 < nfull) load_scales(kt + 1, sa_next, sb_next);
    compute_tile(lds + stage * STAGE);
    rotate_scales();
    stage = stage + 1 == NS ? 0 : stage + 1;
    fill = fill + 1 == NS ? 0 : fill + 1;
  }
  // K tail (K bytes % RBK != 0): one more tile, zero-filled past K, outside the pipelined loop.
  // (Block-scaled operands: whole scale blocks; the scales of the blocks past K read as 2^0.)
  if (nfull * RBK < p.k_bytes) {
    block_barrier();  // every wave is done with the ring
    guarded_tile(nfull, lds);
    if constexpr (Cfg::kScaled) {
      const int nblocks = (p.k_bytes - nfull * RBK) / Cfg::kBlockBytes;
#pragma unroll
      for (int t = 0; t < MT; t++) {
        int r = min(m0 + wm * TM + t * 32 + l32, p.M - 1);
        sa[t] = Cfg::load_scale_tail(p.sA + (int64_t)r * p.lds_a, nfull, g, nblocks);
      }
#pragma unroll
      for (int t = 0; t < NT; t++) {
        int r = min(n0 + wn * TN + t * 32 + l32, p.N - 1);
        sb[t] = Cfg::load_scale_tail(p.sB + (int64_t)r * p.lds_b, nfull, g, nblocks);
      }
    }
    wait_all();
    __syncthreads();
    compute_tile(lds);
  }

  gemm_epilogue<MT, NT>(acc, p, m0 + wm * TM, n0 + wn * TN, l32, g);
}

template <typename Cfg, int BM, int BN, int WM, int WN, bool B_KMAJOR, int NS>
__global__ __launch_bounds__(WM * WN * 64, 1) void gemm_kernel(GemmArgs p) {
  // ring of NS LDS stages (dynamic LDS: NS * STAGE bytes at launch)
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  const int num_m = (p.M + BM - 1) / BM, num_n = (p.N + BN - 1) / BN;
  int pid = xcd_remap(blockIdx.x, num_m * num_n);
  int pm, pn;
  grouped_tile(pid, num_m, num_n, p.group_m, pm, pn);
  gemm_tile_body<Cfg, BM, BN, WM, WN, B_KMAJOR, NS>(p, pm, pn, (LDS_PTR(char))smem);
}

// Split-K for products of few tiles with a long K (one row of tiles against a long weight, a small square against a
// long K): workgroup z * tiles + t multiplies the K bytes [z * chunk, z * chunk + chunk) of tile t and leaves the fp32
// partial tile in slice z of the workspace ([splits][M][N] floats); splitk_reduce_kernel adds the slices and does the
// epilogue.  The one-workgroup-per-tile kernel keeps two to four K steps of loads in flight per workgroup, which with
// a handful of workgroups is a small fraction of what the memory system needs to be busy.
template <typename Cfg, int BM, int BN, int WM, int WN, bool B_KMAJOR, int NS>
__global__ __launch_bounds__(WM * WN * 64, 1) void gemm_splitk_kernel(GemmArgs p, int chunk_bytes) {
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  const int num_m = (p.M + BM - 1) / BM, num_n = (p.N + BN - 1) / BN, tiles = num_m * num_n;
  const int z = blockIdx.x / tiles;
  int pm, pn;
  grouped_tile(xcd_remap(blockIdx.x % tiles, tiles), num_m, num_n, p.group_m, pm, pn);
  GemmArgs q = p;
  const int k0 = z * chunk_bytes;
  q.k_bytes = p.k_bytes - k0 < chunk_bytes ? p.k_bytes - k0 : chunk_bytes;   // (the host leaves no split empty)
  q.K = q.k_bytes / Cfg::kElemBytes;
  q.A = p.A + k0;
  q.B = B_KMAJOR ? p.B + k0 : p.B + (int64_t)(k0 / Cfg::kElemBytes) * p.ldb;
  q.C = (char*)(p.workspace + (int64_t)z * p.M * p.N);
  q.ldc = p.N; q.scn = 1; q.out_dtype = 4;   // fp32 partial sums, dense rows
  q.c_vec_ok = p.N % 4 == 0;                 // (the workspace is 16-byte aligned)
  q.a_scale = nullptr; q.b_scale = nullptr; q.activation = 0; q.aux = nullptr;
  gemm_tile_body<Cfg, BM, BN, WM, WN, B_KMAJOR, NS>(q, pm, pn, (LDS_PTR(char))smem);
}

template <typename Cfg, bool B_KMAJOR>
static int launch_gemm_splitk(const GemmArgs& p, int splits, int chunk_bytes, hipStream_t stream) {
  constexpr int BM = 128, BN = 128, NS = 4;
  constexpr int smem = NS * (BM + BN) * RBK;
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)gemm_splitk_kernel<Cfg, BM, BN, 2, 2, B_KMAJOR, NS>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) return (int)e;
    attr_set = true;
  }
  const int tiles = ((p.M + BM - 1) / BM) * ((p.N + BN - 1) / BN);
  gemm_splitk_kernel<Cfg, BM, BN, 2, 2, B_KMAJOR, NS><<<dim3(tiles * splits), dim3(256), smem, stream>>>(p, chunk_bytes);
  return (int)hipGetLastError();
}

// ---------------------------------------------------------------------------------------------
// Grouped GEMM: a fixed number of workgroups walks the tiles of `group_size` independent
// problems C_g = A_g @ B_g, whose pointers, sizes and leading dimensions live in device arrays -
// the contract of the reference's `grouped_matmul_kernel`
// (python/tutorials/08-grouped-gemm.py:64-140): tiles are numbered problem after problem, row
// major inside a problem, and program b takes tiles b, b + nprog, b + 2 nprog, ...
// Here b is first remapped so that the programs of one XCD take neighbouring tiles (shared A
// panels stay in one L2), a tile is the 128x128 MFMA tile above with its edge handling (the
// reference assumes full tiles), and a problem whose leading dimensions or N, K are not multiples
// of 8 elements - no 16-byte rows - is computed by a plain dot-product loop instead.
// ---------------------------------------------------------------------------------------------
// Two instantiations are launched back to back: 256x256 tiles (eight waves, one program per CU) and
// 128x128 tiles (four waves, two programs per CU).  Both scan the size table first and only one of
// them works: the large tiles when the group holds at least `big_tiles_min` of them (enough to give
// every CU one), the small tiles otherwise - a decision every workgroup of both launches reaches
// alike from the same table, so no host round trip is needed to see sizes that live on the device.
//
// A third launch (gemm_wave128.hip) takes groups made of whole 256x256 tiles only, see grouped_plan.

// Which grouped kernel computes this group: 2 = the four-wave 16x16-MFMA kernel (every problem whole
// 256x256 tiles, K a multiple of 128 and at least `wave128_min_k`, 16-byte rows of A, 512-byte multiples
// as pitch of B, 32-bit lane offsets, and at least `big_tiles_min` tiles), 1 = 256x256 tiles,
// 0 = 128x128 tiles.  (That kernel restarts its two-stage pipeline at every run of tiles and fetches two K steps
// too many per run; measured against the other two on fp16 groups of 256 to 2048 tiles of 1024^2 to 4096^2
// problems it gains 5-25 % with K from 512 to 4096.)
// Every wave reads the tables with one problem per lane (all loads in flight at once: a serial scan of 16
// problems took 4-8 us in each of the three launches) and combines the lanes' findings.
__device__ __forceinline__ int grouped_plan(const GroupedArgs& ga, long long* total_tiles = nullptr) {
  long long big_tiles = 0;
  bool whole = true;
  for (int gi = threadIdx.x & 63; gi < ga.group_size; gi += 64) {
    const int gm = ga.sizes[gi * 3], gn = ga.sizes[gi * 3 + 1], gk = ga.sizes[gi * 3 + 2];
    const int lda = ga.lds[gi * 3], ldb = ga.lds[gi * 3 + 1];
    big_tiles += (long long)((gm + 255) / 256) * ((gn + 255) / 256);
    whole = whole && gm % 256 == 0 && gn % 256 == 0 && gk % 128 == 0 && gk >= 128 && gk >= ga.wave128_min_k && lda % 8 == 0 && ldb % 256 == 0 &&
            lda > 0 && ldb > 0 && (ga.a_ptrs[gi] | ga.b_ptrs[gi]) % 16 == 0 &&
            (int64_t)lda * 16 + gk * 2 < (1ll << 31) && (int64_t)gk * ldb * 2 + 512 < (1ll << 31);
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) big_tiles += __shfl_xor(big_tiles, off);
  if (total_tiles) *total_tiles = __builtin_amdgcn_readfirstlane((int)big_tiles);   // (256x256 tiles of all problems)
  const bool all_whole = ga.wave128_min_k > 0 && __all(whole);
  const int plan = (all_whole && big_tiles >= ga.big_tiles_min) ? 2 : (big_tiles >= ga.big_tiles_min ? 1 : 0);
  return __builtin_amdgcn_readfirstlane(plan);
}

template <typename Cfg, typename T, int BM, int BN, int WM, int WN>
__global__ __launch_bounds__(WM * WN * 64, 1) void gemm_grouped_kernel(GroupedArgs ga) {
  constexpr int NS = 4;
  constexpr bool BIG = BM == 256;
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  LDS_PTR(char) const lds = (LDS_PTR(char))smem;
  if (grouped_plan(ga) != (BIG ? 1 : 0)) return;
  const int nprog = gridDim.x;
  int tile_idx = xcd_remap(blockIdx.x, nprog);
  int last_problem_end = 0;
  for (int gi = 0; gi < ga.group_size; gi++) {
    const int gm = ga.sizes[gi * 3], gn = ga.sizes[gi * 3 + 1], gk = ga.sizes[gi * 3 + 2];
    const int num_m = (gm + BM - 1) / BM, num_n = (gn + BN - 1) / BN;
    const int num_tiles = num_m * num_n;
    if (tile_idx >= last_problem_end && tile_idx < last_problem_end + num_tiles) {
      const int lda = ga.lds[gi * 3], ldb = ga.lds[gi * 3 + 1], ldc = ga.lds[gi * 3 + 2];
      GemmArgs p{};
      p.A = (const char*)ga.a_ptrs[gi]; p.B = (const char*)ga.b_ptrs[gi]; p.C = (char*)ga.c_ptrs[gi];
      p.M = gm; p.N = gn; p.K = gk; p.k_bytes = gk * 2;
      p.lda = (int64_t)lda * 2; p.ldb = (int64_t)ldb * 2; p.ldc = ldc; p.scn = 1;
      p.out_dtype = ga.out_dtype; p.group_m = 1;
      p.c_vec_ok = (ldc % 4 == 0) && (((uintptr_t)p.C) % 16 == 0);
      p.lean_ok = 1;
      const bool rows16 = ((lda | ldb | gn | gk) % 8 == 0) && ((((uintptr_t)p.A) | ((uintptr_t)p.B)) % 16 == 0);
      while (tile_idx >= last_problem_end && tile_idx < last_problem_end + num_tiles) {
        const int t = tile_idx - last_problem_end;
        const int pm = t / num_n, pn = t % num_n;
        if (rows16) {
          gemm_tile_body<Cfg, BM, BN, WM, WN, false, NS>(p, pm, pn, lds);
          // the next tile refills the ring: every wave must be done reading it
          wait_all();
          __syncthreads();
        } else {
          const T* A = (const T*)p.A;
          const T* B = (const T*)p.B;
          T* C = (T*)p.C;
          for (int e = threadIdx.x; e < BM * BN; e += WM * WN * 64) {
            const int m = pm * BM + e / BN, n = pn * BN + e % BN;
            if (m < gm && n < gn) {
              float acc = 0.f;
              for (int k = 0; k < gk; k++) acc = fmaf((float)A[(int64_t)m * lda + k], (float)B[(int64_t)k * ldb + n], acc);
              C[(int64_t)m * ldc + n] = (T)acc;
            }
          }
        }
        tile_idx += nprog;
      }
    }
    last_problem_end += num_tiles;
  }
}

template <typename Cfg, typename T, int BM, int BN, int WM, int WN>
static int launch_gemm_grouped_one(const GroupedArgs& ga, int nprog, hipStream_t stream) {
  constexpr int smem = 4 * (BM + BN) * RBK;
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)gemm_grouped_kernel<Cfg, T, BM, BN, WM, WN>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) return (int)e;
    attr_set = true;
  }
  gemm_grouped_kernel<Cfg, T, BM, BN, WM, WN><<<dim3(nprog), dim3(WM * WN * 64), smem, stream>>>(ga);
  return (int)hipGetLastError();
}

// nprog: programs of the 128x128 form; nprog_big: programs of the 256x256 form (one per CU)
template <typename Cfg, typename T>
static int launch_gemm_grouped(const GroupedArgs& ga, int nprog, int nprog_big, hipStream_t stream) {
  int rc = ga.wave128_min_k > 0 ? gemm_wave128_grouped_launch(ga, std::is_same<T, __bf16>::value, nprog_big, stream) : 0;
  if (rc) return rc;
  rc = launch_gemm_grouped_one<Cfg, T, 256, 256, 2, 4>(ga, nprog_big, stream);
  if (rc) return rc;
  return launch_gemm_grouped_one<Cfg, T, 128, 128, 2, 2>(ga, nprog, stream);
}

// ---------------------------------------------------------------------------------------------
// Ping-pong variant for the 8-wave tiles.  With one barrier per K step all eight waves stall,
// issue loads and wait for their first LDS reads at the same time, and the MFMA pipes idle
// meanwhile.  Here the two waves that share a SIMD (wave w and wave w+4) run half a step apart:
// every K step of a wave is a MEMORY phase (issue its share of the direct loads for the tile
// NS-1 steps ahead, read ALL operands of the current tile from LDS into registers) and a
// COMPUTE phase (nothing but MFMAs), separated by workgroup barriers.  Waves 4-7 execute one
// extra barrier before their loop and waves 0-3 one after, so at every barrier one wave of each
// SIMD arrives from MFMAs and the other from memory work.
//
// Hazards:  a stage is refilled (tile kt+NS-1 into the stage of tile kt-1) in MEM(kt); waves 0-3
// do that in phase 2kt, after the barrier that ended waves 4-7's MEM(kt-1), the last reader of
// tile kt-1.  Tile kt is first read in phase 2kt; every wave waits for its own share of tile kt
// before the barrier that ends phase 2kt-1 (waves 0-3 at the end of COMPUTE(kt-1), waves 4-7 at
// the end of MEM(kt-1)), leaving its NS-2 younger shares in flight.
//
// Block scales (MX) travel with the tile: every wave copies 64 rows x 4 scale bytes per step
// with a 4-byte direct load (waves 0-3 the A rows, waves 4-7 the B rows).
// ---------------------------------------------------------------------------------------------
template <typename Cfg, int BM, int BN, bool B_KMAJOR, int NS>
__global__ __launch_bounds__(512, 1) void gemm_pp_kernel(GemmArgs p) {
  using Operand = typename Cfg::Operand;
  constexpr int WM = 2, WN = 4, NW = 8, TM = BM / WM, TN = BN / WN, MT = TM / 32, NT = TN / 32;
  constexpr int A_BYTES = BM * RBK, B_BYTES = BN * RBK;
  constexpr int SC_BYTES = Cfg::kScaled ? (BM + BN) * 4 : 0;
  constexpr int STAGE = A_BYTES + B_BYTES + SC_BYTES;
  constexpr int KS = Cfg::kSteps, NC = Cfg::kChunks;
  static_assert(B_KMAJOR || (Cfg::kRowMajorB && Cfg::kElemBytes == 2), "row-major B: the 16-bit transpose read only in this kernel");
  static_assert(!Cfg::kScaled || (BM == 256 && BN == 256), "scale copies assume 64 rows per wave");
  using CopyA = TileCopyK<BM, NW>;
  using CopyBk = TileCopyK<BN, NW>;
  using CopyBn = TileCopyKN<BN, NW>;
  constexpr int ITA = CopyA::kIters;
  constexpr int ITB = B_KMAJOR ? CopyBk::kIters : CopyBn::kIters;
  constexpr int KROWS = RBK / 2;
  constexpr int kShare = ITA + ITB + (Cfg::kScaled ? 1 : 0);  // direct loads per wave and tile

  extern __shared__ __attribute__((aligned(1024))) char smem[];
  LDS_PTR(char) const lds = (LDS_PTR(char))smem;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WN, wn = wave % WN;
  // the half of the waves that runs one phase behind (kept in a scalar register: the barriers
  // below must be skipped by a real branch)
  const bool late = __builtin_amdgcn_readfirstlane(tid) >= 256;

  const int num_m = (p.M + BM - 1) / BM, num_n = (p.N + BN - 1) / BN;
  int pid = xcd_remap(blockIdx.x, num_m * num_n);
  int pm, pn;
  grouped_tile(pid, num_m, num_n, p.group_m, pm, pn);
  const int m0 = pm * BM, n0 = pn * BN;

  const char* srcA[ITA];
  const char* srcB[ITB];
#pragma unroll
  for (int i = 0; i < ITA; i++) {
    int r = CopyA::row(wave, lane, i);
    int gr = min(m0 + r, p.M - 1);
    srcA[i] = p.A + (int64_t)gr * p.lda + CopyA::chunk(lane, r) * 16;
  }
#pragma unroll
  for (int i = 0; i < ITB; i++) {
    if constexpr (B_KMAJOR) {
      int r = CopyBk::row(wave, lane, i);
      int gr = min(n0 + r, p.N - 1);
      srcB[i] = p.B + (int64_t)gr * p.ldb + CopyBk::chunk(lane, r) * 16;
    } else {
      int r = CopyBn::row(wave, lane, i);
      int n = n0 + CopyBn::col16(lane, r) * 8;
      const int npad = (p.N + 7) / 8 * 8;   // (the last chunk may reach into the row's padding, see gemm_tile_body)
      n = n < npad ? n : npad - 8;
      srcB[i] = p.B + (int64_t)r * p.ldb + (int64_t)n * 2;
    }
  }
  const int64_t stepA = RBK, stepB = B_KMAJOR ? (int64_t)RBK : KROWS * p.ldb;
  // scale rows this lane copies: waves 0-3 rows 64*wave + lane of A, waves 4-7 of B
  const uint8_t* srcS = nullptr;
  if constexpr (Cfg::kScaled) {
    if (!late) srcS = p.sA + (int64_t)min(m0 + wave * 64 + lane, p.M - 1) * p.lds_a;
    else srcS = p.sB + (int64_t)min(n0 + (wave - 4) * 64 + lane, p.N - 1) * p.lds_b;
  }

  auto issue_share = [&](int kt, LDS_PTR(char) a) {
    LDS_PTR(char) b = a + A_BYTES;
#pragma unroll
    for (int i = 0; i < ITA; i++) async_copy16(srcA[i] + kt * stepA, (LDS_PTR(void))(a + (i * NW + wave) * 1024));
#pragma unroll
    for (int i = 0; i < ITB; i++) async_copy16(srcB[i] + kt * stepB, (LDS_PTR(void))(b + (i * NW + wave) * 1024));
    if constexpr (Cfg::kScaled) async_copy4(srcS + Cfg::scale_dword_offset(kt), (LDS_PTR(void))(a + A_BYTES + B_BYTES + wave * 256));
  };

  f32x16 acc[MT][NT];
#pragma unroll
  for (int i = 0; i < MT; i++)
#pragma unroll
    for (int j = 0; j < NT; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

  const int l32 = lane & 31, g = lane >> 5;
  const int i16 = lane & 15, q = lane >> 4;
  unsigned offA[KS][NC], offB[KS][NC];
#pragma unroll
  for (int ks = 0; ks < KS; ks++)
#pragma unroll
    for (int c = 0; c < NC; c++) {
      offA[ks][c] = kmajor_off(wm * TM + l32, Cfg::chunk(ks, g, c));
      offB[ks][c] = A_BYTES + kmajor_off(wn * TN + l32, Cfg::chunk(ks, g, c));
    }
  unsigned offBn[NT];
  {
    int k = (q >> 1) * 8 + (i16 >> 2);
#pragma unroll
    for (int t = 0; t < NT; t++) {
      int c32 = (wn * TN + t * 32) / 16 + (q & 1);
      offBn[t] = A_BYTES + k * (BN * 2) + ((c32 ^ ((k & 3) << 1)) << 5) + (i16 & 3) * 8;
    }
  }
  const unsigned offSA = A_BYTES + B_BYTES + (wm * TM + l32) * 4;
  const unsigned offSB = A_BYTES + B_BYTES + BM * 4 + (wn * TN + l32) * 4;

  Operand fa[KS][MT], fb[KS][NT];
  int sa[MT], sb[NT];
  auto read_tile = [&](unsigned base, int kt) {
    static_for<KS>([&](auto KS_) {
      constexpr int ks = decltype(KS_)::value;
      static_for<MT>([&](auto T_) {
        constexpr int t = decltype(T_)::value;
        if constexpr (NC == 1) {
          fa[ks][t] = __builtin_bit_cast(Operand, lds_read_b128<t * 32 * RBK>(base + offA[ks][0]));
        } else {
          i32x4 lo = lds_read_b128<t * 32 * RBK>(base + offA[ks][0]);
          i32x4 hi = lds_read_b128<t * 32 * RBK>(base + offA[ks][1]);
          fa[ks][t] = __builtin_bit_cast(Operand, (i32x8)__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
        }
      });
      static_for<NT>([&](auto T_) {
        constexpr int t = decltype(T_)::value;
        if constexpr (!B_KMAJOR) {
          constexpr int imm = ks * 16 * BN * 2;
          i32x2 lo = lds_read_tr16_b64<imm>(base + offBn[t]);
          i32x2 hi = lds_read_tr16_b64<imm + 4 * BN * 2>(base + offBn[t]);
          fb[ks][t] = __builtin_bit_cast(Operand, (i32x4)__builtin_shufflevector(lo, hi, 0, 1, 2, 3));
        } else if constexpr (NC == 1) {
          fb[ks][t] = __builtin_bit_cast(Operand, lds_read_b128<t * 32 * RBK>(base + offB[ks][0]));
        } else {
          i32x4 lo = lds_read_b128<t * 32 * RBK>(base + offB[ks][0]);
          i32x4 hi = lds_read_b128<t * 32 * RBK>(base + offB[ks][1]);
          fb[ks][t] = __builtin_bit_cast(Operand, (i32x8)__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
        }
      });
    });
    if constexpr (Cfg::kScaled) {
      static_for<MT>([&](auto T_) { constexpr int t = decltype(T_)::value; sa[t] = lds_read_b32<t * 128>(base + offSA); });
      static_for<NT>([&](auto T_) { constexpr int t = decltype(T_)::value; sb[t] = lds_read_b32<t * 128>(base + offSB); });
    }
    lds_wait<0>();
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
#pragma unroll
      for (int t = 0; t < MT; t++) lds_use(fa[ks][t]);
#pragma unroll
      for (int t = 0; t < NT; t++) lds_use(fb[ks][t]);
    }
    if constexpr (Cfg::kScaled) {
#pragma unroll
      for (int t = 0; t < MT; t++) { lds_use(sa[t]); sa[t] = Cfg::scale_fixup(sa[t], kt, g); }
#pragma unroll
      for (int t = 0; t < NT; t++) { lds_use(sb[t]); sb[t] = Cfg::scale_fixup(sb[t], kt, g); }
    }
  };
  auto multiply_tile = [&]() {
    static_for<KS>([&](auto KS_) {
      constexpr int ks = decltype(KS_)::value;
#pragma unroll
      for (int i = 0; i < MT; i++)
#pragma unroll
        for (int j = 0; j < NT; j++) {
          if constexpr (Cfg::kScaled) acc[i][j] = Cfg::template mma<ks>(fb[ks][j], fa[ks][i], acc[i][j], sb[j], sa[i]);
          else acc[i][j] = Cfg::template mma<ks>(fb[ks][j], fa[ks][i], acc[i][j], 0, 0);
        }
    });
  };
  auto phase_barrier = [&]() {
    __builtin_amdgcn_sched_barrier(0);
    block_barrier();
    __builtin_amdgcn_sched_barrier(0);
  };
  // wait for this wave's share of tile `next`, given that shares up to tile `issued_upto` are out
  auto wait_share = [&](int next_plus, int nfull) {
    // called with next_plus = j + NS - 1 where j is the current step: in steady state NS-2
    // younger shares stay in flight, near the end of K everything is awaited
    if (next_plus < nfull) wait_vmcnt<(NS - 2) * kShare>(); else wait_vmcnt<0>();
  };

  const int nfull = p.k_bytes / RBK;
#pragma unroll
  for (int s = 0; s < NS - 1; s++)
    if (s < nfull) issue_share(s, lds + s * STAGE);
  if (NS - 1 <= nfull) wait_vmcnt<(NS - 2) * kShare>(); else wait_vmcnt<0>();
  phase_barrier();            // tile 0 is in LDS
  if (late) phase_barrier();  // waves 4-7 start one phase later

  int stage = 0, fill = NS - 1;
  for (int kt = 0; kt < nfull; kt++) {
    // ---- memory phase
    if (kt + NS - 1 < nfull) issue_share(kt + NS - 1, lds + fill * STAGE);
    read_tile(lds_addr(lds + stage * STAGE), kt);
    if (late) wait_share(kt + NS - 1, nfull);
    phase_barrier();
    // ---- compute phase
    multiply_tile();
    if (!late) wait_share(kt + NS - 1, nfull);
    phase_barrier();
    stage = stage + 1 == NS ? 0 : stage + 1;
    fill = fill + 1 == NS ? 0 : fill + 1;
  }
  if (!late) phase_barrier();  // waves 0-3 catch up: every wave has executed the same number of barriers

  gemm_epilogue<MT, NT>(acc, p, m0 + wm * TM, n0 + wn * TN, l32, g);
}

// Stream-K partition: `ntiles * groups_per_tile` groups of K steps dealt evenly to `nprog` programs;
// program `id` gets the half-open range [lo, hi) of global group indices (tile = index / groups_per_tile).
struct StreamKRange { long lo, hi; };
__host__ __device__ inline StreamKRange streamk_range(int ntiles, int groups_per_tile, int nprog, int id) {
  const long total = (long)ntiles * groups_per_tile;
  const long per = total / nprog, rem = total % nprog;
  const long lo = id * per + (id < rem ? id : rem);
  return {lo, lo + per + (id < rem ? 1 : 0)};
}
__host__ __device__ inline int streamk_owner(int ntiles, int groups_per_tile, int nprog, long group) {
  const long total = (long)ntiles * groups_per_tile;
  const long per = total / nprog, rem = total % nprog;
  const long big = rem * (per + 1);
  return group < big ? (int)(group / (per + 1)) : (int)(rem + (group - big) / per);
}

// Second kernel of stream-K: one 64-lane workgroup per 32x32 MFMA sub-tile of C (64 per 256x256 tile,
// so that even a handful of split tiles spreads over the device).  A tile that several programs
// covered in parts is summed from their workspace slots (in program order: deterministic) and
// stored through the usual epilogue; tiles one program covered alone were stored by it already.
// Workspace layout of a partial tile: [wave][i][j][lane][16 accumulator registers], i.e. 64 bytes per
// lane and sub-tile, written and read with 16-byte accesses.
template <int WN>
__global__ __launch_bounds__(64) void gemm_streamk_fixup_kernel(GemmArgs p, int nprog, int groups_per_tile) {
  constexpr int BM = 256, BN = 256, WM = 2, NW = WM * WN, TM = BM / WM, TN = BN / WN, MT = TM / 32, NT = TN / 32;
  constexpr int SUB = NW * MT * NT;  // 32x32 sub-tiles per tile
  const int num_m = (p.M + BM - 1) / BM, num_n = (p.N + BN - 1) / BN;
  const int t = blockIdx.x / SUB, sub = blockIdx.x % SUB;
  const int first = streamk_owner(num_m * num_n, groups_per_tile, nprog, (long)t * groups_per_tile);
  const int last = streamk_owner(num_m * num_n, groups_per_tile, nprog, (long)(t + 1) * groups_per_tile - 1);
  if (first == last) return;
  const int lane = threadIdx.x;
  const int wave = sub / (MT * NT), i = (sub / NT) % MT, j = sub % NT;
  const int wm = wave / WN, wn = wave % WN, l32 = lane & 31, g = lane >> 5;
  f32x4 sum[4];
#pragma unroll
  for (int q = 0; q < 4; q++) sum[q] = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int prog = first; prog <= last; prog++) {
    const StreamKRange r = streamk_range(num_m * num_n, groups_per_tile, nprog, prog);
    const int slot = (int)(r.lo / groups_per_tile) == t ? 0 : 1;
    const f32x4* ws = (const f32x4*)(p.workspace + ((int64_t)prog * 2 + slot) * (BM * BN) + (int64_t)sub * 1024 + lane * 16);
#pragma unroll
    for (int q = 0; q < 4; q++) sum[q] += ws[q];
  }
  f32x16 acc[1][1];
#pragma unroll
  for (int r = 0; r < 16; r++) acc[0][0][r] = sum[r >> 2][r & 3];
  int pm, pn;
  grouped_tile(t, num_m, num_n, p.group_m, pm, pn);
  gemm_epilogue<1, 1>(acc, p, pm * BM + wm * TM + i * 32, pn * BN + wn * TN + j * 32, l32, g);
}

// ---------------------------------------------------------------------------------------------
// Software-pipelined variant of the 256x256 tile, four or eight waves.  With four: one wave per SIMD, each owning a 128x128 quarter of C
// (256 accumulator registers).  Per K step a wave reads (4 + 4) x 32 operand rows from LDS for
// 32 MFMAs - two thirds of the LDS traffic per flop of the 128x64 wave tiles above - and, with
// no second wave on the SIMD to hide latencies, everything is software pipelined inside the wave:
//   * direct loads run NS tiles ahead (tile kt+NS goes into the stage tile kt just vacated);
//   * ALL operands of tile kt+1 are read from LDS into a second register set while the MFMAs of
//     tile kt issue; the reads and the direct loads of a step are spread over the first MFMAs of
//     the step, one or two per MFMA, in program order (scheduling barriers keep them there);
//   * one barrier per step, at its top: by then every wave holds tile kt in registers (so its
//     stage may be overwritten) and has seen its own share of tile kt+1 arrive;
//   * between the MFMAs of the K loop there are LDS reads, direct loads and scalar bookkeeping
//     only: the loads take a scalar tile base plus a fixed 32-bit lane offset, the ring stage
//     enters the LDS reads as an immediate (the loop is unrolled over the ring);
//   * PERSIST: one workgroup per CU walks several tiles as one stream of K steps (see below);
//     otherwise one tile per workgroup, and a partial last K step is finished through a masked
//     register path.
// ---------------------------------------------------------------------------------------------
template <typename Cfg, int WN, bool B_KMAJOR, int NS, bool PERSIST = false, bool SK = false>
__global__ __launch_bounds__(2 * WN * 64, 1) void gemm_w4_kernel(GemmArgs p) {
  static_assert(!PERSIST || WN == 4, "the persistent form is the eight-wave one");
  static_assert(!SK || (PERSIST && !Cfg::kScaled), "stream-K builds on the persistent form of the unscaled types");
  using Operand = typename Cfg::Operand;
  constexpr int BM = 256, BN = 256, WM = 2, NW = WM * WN, TM = BM / WM, TN = BN / WN, MT = TM / 32, NT = TN / 32;
  static_assert(WN == 2 || WN == 4, "four or eight waves");
  constexpr int A_BYTES = BM * RBK, B_BYTES = BN * RBK;
  constexpr int STAGE = A_BYTES + B_BYTES;
  // block scales: 16 bytes per row (SPG K steps) at a time into a two-slot ring behind the tiles
  constexpr int SPG = 4 * Cfg::kStepsPerScaleDword;
  constexpr int SC_SLOT = (BM + BN) * 16;
  constexpr int KS = Cfg::kSteps, NC = Cfg::kChunks;
  static_assert(B_KMAJOR || (Cfg::kRowMajorB && Cfg::kElemBytes == 2), "row-major B: the 16-bit transpose read only in this kernel");
  using CopyA = TileCopyK<BM, NW>;
  using CopyBk = TileCopyK<BN, NW>;
  using CopyBn = TileCopyKN<BN, NW>;
  constexpr int ITA = CopyA::kIters;
  constexpr int ITB = B_KMAJOR ? CopyBk::kIters : CopyBn::kIters;
  constexpr int KROWS = RBK / 2;
  constexpr int kShare = ITA + ITB;               // direct loads per wave and tile

  extern __shared__ __attribute__((aligned(1024))) char smem[];
  LDS_PTR(char) const lds = (LDS_PTR(char))smem;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // scalar: LDS destinations of the direct loads are scalar math
  const int wm = wave / WN, wn = wave % WN;

  // One tile per workgroup, or (PERSIST, the schedule of python/tutorials/09-persistent-matmul.py:
  // 141-190) gridDim.x workgroups that each walk tiles lid, lid + G, lid + 2G, ... of the grouped
  // order as ONE stream of K steps: the direct loads run NS steps ahead across tile boundaries, so
  // the ring never drains between tiles.  lid keeps the workgroups of one XCD on neighbouring tiles.
  // SK (stream-K): the G programs instead split ALL K steps of ALL tiles evenly (in groups of NS
  // steps, tiles in the grouped order): program lid walks one contiguous range of the global step
  // sequence, which may begin and end in the middle of a tile.  A tile it covers completely is
  // stored as usual; of a tile it covers partly it leaves the fp32 partial sums in the workspace
  // (slot 0 = the tile its range begins in, slot 1 = the tile it ends in) and a second kernel adds
  // the partial tiles up.  No program ever waits for another one.
  const int num_m = (p.M + BM - 1) / BM, num_n = (p.N + BN - 1) / BN;
  const int ntiles = num_m * num_n;
  const int G = PERSIST ? (int)gridDim.x : ntiles;
  const int lid = xcd_remap(blockIdx.x, G);
  const int nfull = p.k_bytes / RBK;
  int sk_first_tile = 0, sk_kt0 = 0, sk_steps = 0;
  if constexpr (SK) {
    const StreamKRange r = streamk_range(ntiles, nfull / NS, G, lid);
    sk_first_tile = (int)(r.lo / (nfull / NS));
    sk_kt0 = (int)(r.lo % (nfull / NS)) * NS;
    sk_steps = (int)(r.hi - r.lo) * NS;
    if (sk_steps == 0) return;  // more programs than groups of steps
  }
  const int sk_last_tile = SK ? sk_first_tile + (sk_kt0 + sk_steps - 1) / nfull : 0;
  // tiles of this workgroup (PERSIST: the host keeps G <= ntiles) and the q-th of them
  const int ntw = SK ? sk_last_tile - sk_first_tile + 1 : PERSIST ? (ntiles - lid + G - 1) / G : 1;
  auto tile_id = [&](int q) { return SK ? sk_first_tile + q : lid + q * G; };
  int pm, pn;
  grouped_tile(tile_id(0), num_m, num_n, p.group_m, pm, pn);
  int m0 = pm * BM, n0 = pn * BN;  // tile being multiplied

  // Sources of the direct loads: a scalar tile base that advances with kt plus a 32-bit per-lane
  // offset that never changes (the host keeps 256 rows of either operand within 2^31 bytes), so a
  // load costs no vector arithmetic.
  // (PERSIST runs on whole tiles only, so the clamps below are neutral and the offsets serve every tile)
  const char* const baseA = p.A + (int64_t)m0 * p.lda;
  const char* const baseB = B_KMAJOR ? p.B + (int64_t)n0 * p.ldb : p.B + (int64_t)n0 * 2;
  unsigned offGA[ITA], offGB[ITB];
#pragma unroll
  for (int i = 0; i < ITA; i++) {
    int r = CopyA::row(wave, lane, i);
    int gr = min(m0 + r, p.M - 1) - m0;
    offGA[i] = (unsigned)gr * (unsigned)p.lda + CopyA::chunk(lane, r) * 16;
  }
#pragma unroll
  for (int i = 0; i < ITB; i++) {
    if constexpr (B_KMAJOR) {
      int r = CopyBk::row(wave, lane, i);
      int gr = min(n0 + r, p.N - 1) - n0;
      offGB[i] = (unsigned)gr * (unsigned)p.ldb + CopyBk::chunk(lane, r) * 16;
    } else {
      int r = CopyBn::row(wave, lane, i);
      int n = n0 + CopyBn::col16(lane, r) * 8;
      const int npad = (p.N + 7) / 8 * 8;   // (the last chunk may reach into the row's padding, see gemm_tile_body)
      n = (n < npad ? n : npad - 8) - n0;
      offGB[i] = (unsigned)r * (unsigned)p.ldb + (unsigned)n * 2;
    }
  }
  const int64_t stepA = RBK, stepB = B_KMAJOR ? (int64_t)RBK : KROWS * p.ldb;
  // Block scales: a scalar base per tile (first scale row of the tile's A rows / B rows) plus a
  // fixed per-lane row offset, like the operand loads.  Four waves: every wave copies 64 A rows and
  // 64 B rows; eight waves: waves 0-3 the A rows, waves 4-7 the B rows (the LDS side is A scales
  // then B scales, 256 bytes per wave either way) - `scA` then is the one base the wave needs.
  // (Edge tiles clamp rows onto the last one; PERSIST runs on whole tiles, where that is neutral.)
  const uint8_t* scA = nullptr;
  const uint8_t* scB = nullptr;
  const uint8_t* scA_next = nullptr;  // PERSIST: the same base in the workgroup's next tile
  unsigned scoffA = 0, scoffB = 0;
  const bool second_half_wave = NW == 8 && wave >= 4;
  auto scale_base = [&](int tm, int tn, const uint8_t*& a, const uint8_t*& b) {
    a = p.sA + (int64_t)tm * p.lds_a;
    b = p.sB + (int64_t)tn * p.lds_b;
    if (second_half_wave) a = b;
  };
  auto next_tile_scale_base = [&](int q) {  // q: index of a tile of this workgroup (clamped to the last)
    int tm, tn;
    const uint8_t* unused;
    grouped_tile(tile_id(min(q, ntw - 1)), num_m, num_n, p.group_m, tm, tn);
    scale_base(tm * BM, tn * BN, scA_next, unused);
  };
  if constexpr (Cfg::kScaled) {
    const int w4 = wave & 3;
    scoffA = (unsigned)(min(m0 + w4 * 64 + lane, p.M - 1) - m0) * (unsigned)p.lds_a;
    scoffB = (unsigned)(min(n0 + w4 * 64 + lane, p.N - 1) - n0) * (unsigned)p.lds_b;
    if (second_half_wave) scoffA = scoffB;
    scale_base(m0, n0, scA, scB);
    if constexpr (PERSIST) next_tile_scale_base(1);
  }

  // Fill cursor: the (tile, K step) the next direct loads fetch.  It runs NS positions ahead of the
  // multiplication and stops on the last position of the workgroup's stream (which is then fetched
  // again into a dead stage: the number of outstanding loads, and with it the partial waits, stays uniform).
  int ftile = 0, fkt = SK ? sk_kt0 : 0;
  const char* fillA = baseA;
  const char* fillB = baseB;
  auto fill_advance = [&]() {
    if constexpr (PERSIST) fkt++;  // (tile switches happen between groups of NS steps, below)
    else if (fkt + 1 < nfull) fkt++;
  };
  // PERSIST: a tile's K steps are a multiple of NS and the cursor runs NS positions ahead, so it
  // reaches the end of a tile exactly at the end of a group of NS steps: the switch to the next tile
  // (integer divisions of the grouped order) stays out of the step bodies.  After the last tile
  // the cursor wraps onto its first steps, whose re-fetch into dead stages is harmless.
  auto fill_next_tile = [&]() {
    fkt = 0;
    if (ftile + 1 < ntw) {
      ftile++;
      int fm, fn;
      grouped_tile(tile_id(ftile), num_m, num_n, p.group_m, fm, fn);
      fillA = p.A + (int64_t)fm * BM * p.lda;
      fillB = B_KMAJOR ? p.B + (int64_t)fn * BN * p.ldb : p.B + (int64_t)fn * BN * 2;
    }
  };
  // direct load number `i` of this wave's share of the K step at (srcA, srcB)
  auto issue_one = [&](auto I_, const char* srcA, const char* srcB, LDS_PTR(char) a) {
    constexpr int i = decltype(I_)::value;
    if constexpr (i < ITA) {
      async_copy16_sbase(srcA, offGA[i], lds_addr(a) + (i * NW + wave) * 1024);
    } else {
      constexpr int ib = i - ITA;
      async_copy16_sbase(srcB, offGB[ib], lds_addr(a) + A_BYTES + (ib * NW + wave) * 1024);
    }
  };
  // scale group sg (the 16 scale bytes per row of K steps sg*SPG ..) into ring slot sg % 2: one
  // direct load moves 64 rows; past the last group the last one is fetched again
  LDS_PTR(char) const sc_ring = lds + NS * STAGE;
  const int ngroups = p.k_bytes / (RBK * SPG);
  // Scale groups are numbered along the workgroup's whole stream of K steps (`gcount` = the group of
  // the step being multiplied); group number n lives in ring slot n % 2.  `sg` = group inside the
  // current tile; past its last group comes group 0 of the next tile (PERSIST) or the last group again.
  int gcount = 0;
  auto issue_scales = [&](int sg, int slot, int tile_index) {
    if constexpr (Cfg::kScaled) {
      const unsigned dst = lds_addr(sc_ring) + slot * SC_SLOT + wave * 1024;
      if (PERSIST && sg >= ngroups && tile_index + 1 < ntw) {
        async_copy16_sbase(scA_next, scoffA, dst);
      } else {
        const int off = min(sg, ngroups - 1) * 16;
        async_copy16_sbase(scA + off, scoffA, dst);
        if constexpr (NW == 4) async_copy16_sbase(scB + off, scoffB, dst + BM * 16);
      }
    }
  };

  f32x16 acc[MT][NT];
#pragma unroll
  for (int i = 0; i < MT; i++)
#pragma unroll
    for (int j = 0; j < NT; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

  const int l32 = lane & 31, g = lane >> 5;
  const int i16 = lane & 15, q = lane >> 4;
  unsigned offA[KS][NC], offB[KS][NC];
#pragma unroll
  for (int ks = 0; ks < KS; ks++)
#pragma unroll
    for (int c = 0; c < NC; c++) {
      offA[ks][c] = kmajor_off(wm * TM + l32, Cfg::chunk(ks, g, c));
      offB[ks][c] = A_BYTES + kmajor_off(wn * TN + l32, Cfg::chunk(ks, g, c));
    }
  unsigned offBn[NT];
  {
    int k = (q >> 1) * 8 + (i16 >> 2);
#pragma unroll
    for (int t = 0; t < NT; t++) {
      int c32 = (wn * TN + t * 32) / 16 + (q & 1);
      offBn[t] = A_BYTES + k * (BN * 2) + ((c32 ^ ((k & 3) << 1)) << 5) + (i16 & 3) * 8;
    }
  }
  const unsigned offSA = (wm * TM + l32) * 16;
  const unsigned offSB = BM * 16 + (wn * TN + l32) * 16;

  // A K step is multiplied in two halves, and the operands of the next half are read from LDS
  // while the MFMAs of the current one issue.  With two MFMA sub-steps per K step (16-bit, fp4)
  // a half is a sub-step: all A and B operands of that sub-step.  With one sub-step (fp8) a half
  // is the upper or lower half of the wave's A rows against all of its B columns; the B
  // operands then live for the whole step and alternate between two register sets by tile parity.
  constexpr bool KSPLIT = KS == 2;
  static_assert(KS == 1 || KS == 2, "one or two MFMA sub-steps per K step");
  constexpr int AH = KSPLIT ? MT : MT / 2;  // A operands per half
  Operand fa[KSPLIT ? 2 : 1][MT], fb[2][NT];
  int sa[MT], sb[NT], sa_in[MT], sb_in[NT];

  // LDS reads of half H of a tile with parity P: A operands, then (K-split: always, M-split: with
  // the first half) the B operands, then with the first half the scale dwords
  auto n_reads = [](int H) constexpr { return AH + ((KSPLIT || H == 0) ? NT : 0) + ((Cfg::kScaled && H == 0) ? MT + NT : 0); };
  // Operand addresses carry the stage as an instruction immediate: the 16-bit offset field reaches
  // two stages, so there are two copies of the per-lane offsets (stages 0-1 and 2-3) and the K loop
  // is unrolled over the ring.
  static_assert(NS == 4 && 2 * STAGE + 3 * 32 * RBK + 16 * BN * 2 + 4 * BN * 2 < 65536 + STAGE, "stage immediates");
  const unsigned lds0 = lds_addr(lds);
  unsigned adrA[2][KS][NC], adrB[2][KS][NC], adrBn[2][NT];
#pragma unroll
  for (int hi = 0; hi < 2; hi++) {
#pragma unroll
    for (int ks = 0; ks < KS; ks++)
#pragma unroll
      for (int c = 0; c < NC; c++) {
        adrA[hi][ks][c] = lds0 + hi * 2 * STAGE + offA[ks][c];
        adrB[hi][ks][c] = lds0 + hi * 2 * STAGE + offB[ks][c];
      }
#pragma unroll
    for (int t = 0; t < NT; t++) adrBn[hi][t] = lds0 + hi * 2 * STAGE + offBn[t];
  }
  auto read_one = [&](auto R_, auto H_, auto P_, auto STG_, unsigned scbase) {
    constexpr int r = decltype(R_)::value, H = decltype(H_)::value, P = decltype(P_)::value;
    constexpr int hi = decltype(STG_)::value >> 1, SO = (decltype(STG_)::value & 1) * STAGE;
    constexpr int ks = KSPLIT ? H : 0, aset = KSPLIT ? H : 0, bset = KSPLIT ? H : P;
    constexpr int nb = (KSPLIT || H == 0) ? NT : 0;
    if constexpr (r < AH) {
      constexpr int t = (KSPLIT ? 0 : H * AH) + r;
      if constexpr (NC == 1) {
        fa[aset][t] = __builtin_bit_cast(Operand, lds_read_b128<SO + t * 32 * RBK>(adrA[hi][ks][0]));
      } else {
        i32x4 lo4 = lds_read_b128<SO + t * 32 * RBK>(adrA[hi][ks][0]);
        i32x4 hi4 = lds_read_b128<SO + t * 32 * RBK>(adrA[hi][ks][1]);
        fa[aset][t] = __builtin_bit_cast(Operand, (i32x8)__builtin_shufflevector(lo4, hi4, 0, 1, 2, 3, 4, 5, 6, 7));
      }
    } else if constexpr (r < AH + nb) {
      constexpr int u = r - AH;
      if constexpr (!B_KMAJOR) {
        constexpr int imm = SO + ks * 16 * BN * 2;
        i32x2 lo2 = lds_read_tr16_b64<imm>(adrBn[hi][u]);
        i32x2 hi2 = lds_read_tr16_b64<imm + 4 * BN * 2>(adrBn[hi][u]);
        fb[bset][u] = __builtin_bit_cast(Operand, (i32x4)__builtin_shufflevector(lo2, hi2, 0, 1, 2, 3));
      } else if constexpr (NC == 1) {
        fb[bset][u] = __builtin_bit_cast(Operand, lds_read_b128<SO + u * 32 * RBK>(adrB[hi][ks][0]));
      } else {
        i32x4 lo4 = lds_read_b128<SO + u * 32 * RBK>(adrB[hi][ks][0]);
        i32x4 hi4 = lds_read_b128<SO + u * 32 * RBK>(adrB[hi][ks][1]);
        fb[bset][u] = __builtin_bit_cast(Operand, (i32x8)__builtin_shufflevector(lo4, hi4, 0, 1, 2, 3, 4, 5, 6, 7));
      }
    } else {
      constexpr int t = r - AH - nb;
      if constexpr (t < MT) sa_in[t] = lds_read_b32<t * 512>(scbase + offSA);
      else sb_in[t - MT] = lds_read_b32<(t - MT) * 512>(scbase + offSB);
    }
  };
  // after the reads of a half have been waited for: tie the registers to the wait; with the
  // first half of a tile come its scales
  auto settle = [&](auto H_, auto P_, int kt) {
    constexpr int H = decltype(H_)::value, P = decltype(P_)::value;
    constexpr int aset = KSPLIT ? H : 0, bset = KSPLIT ? H : P, alo = KSPLIT ? 0 : H * AH;
    lds_wait<0>();
#pragma unroll
    for (int t = 0; t < AH; t++) lds_use(fa[aset][alo + t]);
    if constexpr (KSPLIT || H == 0) {
#pragma unroll
      for (int t = 0; t < NT; t++) lds_use(fb[bset][t]);
    }
    if constexpr (Cfg::kScaled && H == 0) {
#pragma unroll
      for (int t = 0; t < MT; t++) { lds_use(sa_in[t]); sa[t] = Cfg::scale_fixup(sa_in[t], kt, g); }
#pragma unroll
      for (int t = 0; t < NT; t++) { lds_use(sb_in[t]); sb[t] = Cfg::scale_fixup(sb_in[t], kt, g); }
    }
  };

  constexpr int kMfmas = AH * NT;  // per half

  // MFMAs of half H with the memory instructions of the half in between: the `nreads` LDS reads
  // over the first MFMAs (they are needed at the top of the next half), then the `nloads`
  // direct loads over the rest
  auto half = [&](auto H_, auto P_, auto NREADS_, auto NLOADS_, auto&& memop) {
    constexpr int H = decltype(H_)::value, P = decltype(P_)::value;
    constexpr int nreads = decltype(NREADS_)::value, nloads = decltype(NLOADS_)::value;
    constexpr int ks = KSPLIT ? H : 0, aset = KSPLIT ? H : 0, bset = KSPLIT ? H : P, alo = KSPLIT ? 0 : H * AH;
    constexpr int half_slots = (kMfmas + 1) / 2;
    constexpr int rper = nreads == 0 ? 1 : (nreads + half_slots - 1) / half_slots;
    constexpr int rslots = (nreads + rper - 1) / rper;
    constexpr int lper = nloads == 0 ? 1 : (nloads + (kMfmas - rslots) - 1) / (kMfmas - rslots);
    static_for<kMfmas>([&](auto N_) {
      constexpr int n = decltype(N_)::value, i = alo + n / NT, j = n % NT;
      if constexpr (Cfg::kScaled) acc[i][j] = Cfg::template mma<ks>(fb[bset][j], fa[aset][i], acc[i][j], sb[j], sa[i]);
      else acc[i][j] = Cfg::template mma<ks>(fb[bset][j], fa[aset][i], acc[i][j], 0, 0);
      if constexpr (n < rslots) {
        static_for<rper>([&](auto O_) {
          constexpr int op = rper * n + decltype(O_)::value;
          if constexpr (op < nreads) memop(std::integral_constant<int, op>{});
        });
      } else {
        static_for<lper>([&](auto O_) {
          constexpr int op = (n - rslots) * lper + decltype(O_)::value;
          if constexpr (op < nloads) memop(std::integral_constant<int, nreads + op>{});
        });
      }
      __builtin_amdgcn_sched_barrier(0);
    });
  };

  // prologue: NS tiles in flight (past the end of K the last tile again, which keeps the number
  // of outstanding loads - and with it the partial waits - uniform), first half of tile 0 requested
  issue_scales(0, 0, 0);
#pragma unroll
  for (int s = 0; s < NS; s++) {
    const char* srcA = fillA + fkt * stepA;
    const char* srcB = fillB + fkt * stepB;
    static_for<kShare>([&](auto I_) { issue_one(I_, srcA, srcB, lds + s * STAGE); });
    fill_advance();
  }
  if constexpr (PERSIST) {
    if (fkt == nfull) fill_next_tile();
  }
  wait_vmcnt<(NS - 1) * kShare>();
  __builtin_amdgcn_sched_barrier(0);
  block_barrier();
  __builtin_amdgcn_sched_barrier(0);
  static_for<n_reads(0)>([&](auto R_) { read_one(R_, std::integral_constant<int, 0>{}, std::integral_constant<int, 0>{}, std::integral_constant<int, 0>{}, lds_addr(sc_ring)); });

  // one K step of the tile in ring stage STG (its parity, for the one-sub-step types, is STG % 2);
  // kt = K step inside the current tile
  int ckt = SK ? sk_kt0 : 0, ctile = 0;
  int seg_kt0 = ckt;  // SK: K step at which this program entered the current tile
  auto step = [&](auto STG_) {
    const int kt = ckt;
    constexpr int stage = decltype(STG_)::value, P = stage & 1;
    using H0 = std::integral_constant<int, 0>;
    using H1 = std::integral_constant<int, 1>;
    using P_ = std::integral_constant<int, P>;
    using PN = std::integral_constant<int, P ^ 1>;
    using SN = std::integral_constant<int, (stage + 1) % NS>;
    // ---- first half: multiply it, fetch the second half of the same tile
    settle(H0{}, P_{}, kt);
    half(H0{}, P_{}, std::integral_constant<int, n_reads(1)>{}, std::integral_constant<int, 0>{}, [&](auto OP_) {
      read_one(OP_, H1{}, P_{}, STG_, 0u);
    });
    // ---- second half: every wave holds the whole of tile kt in registers and has seen its own
    //      share of tile kt+1 arrive (NS-2 younger shares stay in flight); after the barrier the
    //      stage of tile kt is refilled with tile kt+NS and the first half of tile kt+1 is fetched
    settle(H1{}, P_{}, kt);
    wait_vmcnt<(NS - 2) * kShare>();
    __builtin_amdgcn_sched_barrier(0);
    block_barrier();
    __builtin_amdgcn_sched_barrier(0);
    // the first step of a scale group fetches the next group: its slot was last read two steps
    // ago, and the loads are older than the NS-2 shares the partial waits leave in flight by the
    // time the group is first read (SPG - 1 >= NS - 1 steps from now)
    if constexpr (Cfg::kScaled) {
      if (kt % SPG == 0) issue_scales(kt / SPG + 1, (gcount + 1) & 1, ctile);
    }
    {
      const int ktn = kt + 1;
      // the next step's scales: same group, or the next one (whose first dword it then reads)
      const bool new_group = ktn % SPG == 0;
      const unsigned scbase = lds_addr(sc_ring) + ((gcount + (new_group ? 1 : 0)) & 1) * SC_SLOT + Cfg::scale_dword_offset(ktn % SPG);
      if (new_group) gcount++;
      LDS_PTR(char) const fill = lds + stage * STAGE;
      const char* srcA = fillA + fkt * stepA;
      const char* srcB = fillB + fkt * stepB;
      constexpr int nr = n_reads(0);
      half(H1{}, P_{}, std::integral_constant<int, nr>{}, std::integral_constant<int, kShare>{}, [&](auto OP_) {
        constexpr int op = decltype(OP_)::value;
        if constexpr (op < nr) read_one(OP_, H0{}, PN{}, SN{}, scbase);
        else issue_one(std::integral_constant<int, op - nr>{}, srcA, srcB, fill);
      });
      fill_advance();
    }
    ckt++;
  };
  const int nsteps_all = SK ? sk_steps : ntw * nfull;
  for (int s = 0; s < nsteps_all; s += NS) {
    step(std::integral_constant<int, 0>{});
    if (s + 1 < nsteps_all) step(std::integral_constant<int, 1>{});
    if (s + 2 < nsteps_all) step(std::integral_constant<int, 2>{});
    if (s + 3 < nsteps_all) step(std::integral_constant<int, 3>{});
    if constexpr (PERSIST) {
      if (fkt == nfull) fill_next_tile();
      // (the host launches this form only when a tile's K steps are a multiple of the ring length, so
      //  tiles end here and the epilogue exists once in the loop body)
      if (ckt == nfull || (SK && s + NS >= nsteps_all)) {
        // tile finished: store it, start the next one.  The stores share the vector-memory counter
        // with the direct loads and may complete out of order with them, so the counter is drained
        // once per tile before the partial waits count again (the loads for the next tile's first
        // steps were issued during the last steps of this one and have been in flight since).
        if (SK && (seg_kt0 != 0 || ckt != nfull)) {
          // part of a tile: raw partial sums, register order (the second kernel reads them back alike)
          // ([wave][i][j][lane][16 registers]: 64 bytes per lane and 32x32 sub-tile)
          float* ws = p.workspace + ((int64_t)lid * 2 + (ctile == 0 ? 0 : 1)) * (BM * BN) + lane * 16;
          static_for<MT>([&](auto I_) {
            static_for<NT>([&](auto J_) {
              constexpr int i = decltype(I_)::value, j = decltype(J_)::value;
              f32x4* dst = (f32x4*)(ws + ((wave * MT + i) * NT + j) * 1024);
#pragma unroll
              for (int q = 0; q < 4; q++)
                dst[q] = f32x4{acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
            });
          });
        } else {
          gemm_epilogue<MT, NT>(acc, p, m0 + wm * TM, n0 + wn * TN, l32, g);
        }
        seg_kt0 = 0;
#pragma unroll
        for (int i = 0; i < MT; i++)
#pragma unroll
          for (int j = 0; j < NT; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;
        ckt = 0;
        ctile++;
        grouped_tile(tile_id(min(ctile, ntw - 1)), num_m, num_n, p.group_m, pm, pn);
        m0 = pm * BM;
        n0 = pn * BN;
        if constexpr (Cfg::kScaled) {
          scA = scA_next;
          next_tile_scale_base(ctile + 1);
        }
        wait_vmcnt<0>();
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }
  // nothing may still be writing this workgroup's LDS when it retires - nor this wave's registers: the last half of
  // the loop has read the operands of a step that does not follow, and the compiler, which sees those registers as
  // written when the read was issued, is free to put the epilogue's values into them ahead of the wait.  Keeping
  // them live across the wait closes that.
  wait_all();
#pragma unroll
  for (int s = 0; s < (KSPLIT ? 2 : 1); s++)
#pragma unroll
    for (int t = 0; t < MT; t++) lds_use(fa[s][t]);
#pragma unroll
  for (int s = 0; s < 2; s++)
#pragma unroll
    for (int t = 0; t < NT; t++) lds_use(fb[s][t]);
  if constexpr (Cfg::kScaled) {
#pragma unroll
    for (int t = 0; t < MT; t++) lds_use(sa_in[t]);
#pragma unroll
    for (int t = 0; t < NT; t++) lds_use(sb_in[t]);
  }

  // Last, partial K step (unscaled types only): its 16-byte chunks past K are written as zeros (the
  // reference masks them to 0, python/tutorials/03-matrix-multiplication.py:297-298).  Goes through
  // registers into stage 0 and is multiplied without overlap: one step out of K / 32.
  if constexpr (!Cfg::kScaled && !PERSIST) {
    if (p.k_bytes % RBK != 0) {
      using Z = std::integral_constant<int, 0>;
      using O = std::integral_constant<int, 1>;
      __syncthreads();  // every wave is done reading the ring
      const int kbase = nfull * RBK;
#pragma unroll
      for (int i = 0; i < ITA; i++) {
        const int r = CopyA::row(wave, lane, i);
        i32x4 v = {0, 0, 0, 0};
        if (kbase + CopyA::chunk(lane, r) * 16 < p.k_bytes) v = *(const i32x4*)(baseA + nfull * stepA + offGA[i]);
        *(LDS_PTR(i32x4))(lds + (i * NW + wave) * 1024 + lane * 16) = v;
      }
#pragma unroll
      for (int i = 0; i < ITB; i++) {
        bool ok;
        if constexpr (B_KMAJOR) ok = kbase + CopyBk::chunk(lane, CopyBk::row(wave, lane, i)) * 16 < p.k_bytes;
        else ok = nfull * KROWS + CopyBn::row(wave, lane, i) < p.K;
        i32x4 v = {0, 0, 0, 0};
        if (ok) v = *(const i32x4*)(baseB + nfull * stepB + offGB[i]);
        *(LDS_PTR(i32x4))(lds + A_BYTES + (i * NW + wave) * 1024 + lane * 16) = v;
      }
      __syncthreads();
      static_for<n_reads(0)>([&](auto R_) { read_one(R_, Z{}, Z{}, Z{}, 0u); });
      settle(Z{}, Z{}, nfull);
      half(Z{}, Z{}, std::integral_constant<int, n_reads(1)>{}, Z{}, [&](auto OP_) { read_one(OP_, O{}, Z{}, Z{}, 0u); });
      settle(O{}, Z{}, nfull);
      half(O{}, Z{}, Z{}, Z{}, [&](auto) {});
    }
  }

  if constexpr (!PERSIST) gemm_epilogue<MT, NT>(acc, p, m0 + wm * TM, n0 + wn * TN, l32, g);
}

template <typename Cfg, int WN, bool B_KMAJOR, int NS, bool PERSIST = false, bool SK = false>
static int launch_gemm_w4(const GemmArgs& p, hipStream_t stream, int num_programs = 0) {
  constexpr int BM = 256, BN = 256;
  constexpr int smem = NS * (BM + BN) * RBK + (Cfg::kScaled ? 2 * (BM + BN) * 16 : 0);
  static_assert(smem <= 160 * 1024, "LDS ring does not fit");
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)gemm_w4_kernel<Cfg, WN, B_KMAJOR, NS, PERSIST, SK>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) return (int)e;
    attr_set = true;
  }
  int num_m = (p.M + BM - 1) / BM, num_n = (p.N + BN - 1) / BN;
  int grid = num_m * num_n;
  if (SK) grid = num_programs;
  else if (PERSIST && num_programs > 0 && num_programs < grid) grid = num_programs;
  gemm_w4_kernel<Cfg, WN, B_KMAJOR, NS, PERSIST, SK><<<dim3(grid), dim3(2 * WN * 64), smem, stream>>>(p);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess || !SK) return (int)e;
  gemm_streamk_fixup_kernel<WN><<<dim3(num_m * num_n * 64), dim3(64), 0, stream>>>(p, grid, (p.k_bytes / RBK) / NS);
  return (int)hipGetLastError();
}

template <typename Cfg, int BM, int BN, bool B_KMAJOR, int NS>
static int launch_gemm_pp(const GemmArgs& p, hipStream_t stream) {
  constexpr int smem = NS * ((BM + BN) * RBK + (Cfg::kScaled ? (BM + BN) * 4 : 0));
  static_assert(smem <= 160 * 1024, "LDS ring does not fit");
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)gemm_pp_kernel<Cfg, BM, BN, B_KMAJOR, NS>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) return (int)e;
    attr_set = true;
  }
  int num_m = (p.M + BM - 1) / BM, num_n = (p.N + BN - 1) / BN;
  gemm_pp_kernel<Cfg, BM, BN, B_KMAJOR, NS><<<dim3(num_m * num_n), dim3(512), smem, stream>>>(p);
  return (int)hipGetLastError();
}

template <typename Cfg, int BM, int BN, int WM, int WN, bool B_KMAJOR, int NS>
static int launch_gemm(const GemmArgs& p, hipStream_t stream) {
  constexpr int smem = NS * (BM + BN) * RBK;
  static_assert(smem <= 160 * 1024, "LDS ring does not fit");
  static bool attr_set = false;  // benign race: setting the attribute twice is harmless
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)gemm_kernel<Cfg, BM, BN, WM, WN, B_KMAJOR, NS>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) return (int)e;
    attr_set = true;
  }
  int num_m = (p.M + BM - 1) / BM, num_n = (p.N + BN - 1) / BN;
  gemm_kernel<Cfg, BM, BN, WM, WN, B_KMAJOR, NS><<<dim3(num_m * num_n), dim3(WM * WN * 64), smem, stream>>>(p);
  return (int)hipGetLastError();
}

// tile: 0 = 256x256 / 8 waves / 4 stages, ping-pong phases (whole K steps only, else tile 2),
//       1 = 128x128 / 4 waves / 4 stages (two workgroups per CU),
//       2 = 256x256 / 8 waves / 4 stages, one barrier per step,
//       3 = 256x256 / 4 waves / 4 stages, software pipelined (whole K steps only, else tile 2),
//       4 = the same pipeline with 8 waves
template <typename Cfg, bool B_KMAJOR>
static int launch_gemm_tile(const GemmArgs& p, int tile, hipStream_t stream) {
  {
    // whole K steps; block scales are fetched 16 bytes per row at a time
    // (the unscaled pipelined kernels finish a partial last K step themselves)
    bool whole = p.k_bytes >= RBK;
    if constexpr (Cfg::kScaled) {
      whole = p.k_bytes % (RBK * 4 * Cfg::kStepsPerScaleDword) == 0 && p.lds_a % 16 == 0 && p.lds_b % 16 == 0 &&
              ((uintptr_t)p.sA | (uintptr_t)p.sB) % 16 == 0;
    }
    {
      // persistent form (5, eight waves; a four-wave persistent form spills): whole tiles, K steps in
      // whole rings, one workgroup per CU; anything else runs the one-tile-per-workgroup form
      const bool stream_ok = whole && p.M % 256 == 0 && p.N % 256 == 0 && p.k_bytes % (4 * RBK) == 0 && p.num_programs > 0;
      if constexpr (!Cfg::kScaled) {
        // 7: stream-K (needs the caller's workspace: two 256x256 fp32 tiles per program)
        if (tile == 7 && stream_ok && p.workspace != nullptr) return launch_gemm_w4<Cfg, 4, B_KMAJOR, 4, true, true>(p, stream, p.num_programs);
      }
      if (tile >= 5 && stream_ok) return launch_gemm_w4<Cfg, 4, B_KMAJOR, 4, true>(p, stream, p.num_programs);
      if (tile >= 5) tile = 4;
    }
    if constexpr (Cfg::kSteps == 2) {  // the four-wave form of the one-sub-step types runs out of registers
      if (tile == 3 && whole) return launch_gemm_w4<Cfg, 2, B_KMAJOR, 4>(p, stream);
    }
    if (tile >= 3 && whole) return launch_gemm_w4<Cfg, 4, B_KMAJOR, 4>(p, stream);
  }
  if (tile >= 3) tile = 2;
  if (tile == 1) return launch_gemm<Cfg, 128, 128, 2, 2, B_KMAJOR, 4>(p, stream);
  if (tile == 0 && p.k_bytes % (RBK * Cfg::kStepsPerScaleDword) == 0) return launch_gemm_pp<Cfg, 256, 256, B_KMAJOR, 4>(p, stream);
  return launch_gemm<Cfg, 256, 256, 2, 4, B_KMAJOR, 4>(p, stream);
}

}  // namespace mi355

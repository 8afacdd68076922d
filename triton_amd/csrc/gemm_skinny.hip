// Skinny GEMM (fp16 / bf16, and fp8 with both operands K-contiguous): one side of the product has at most 64 rows (decode-style M = 16..64,
// or N <= 64), so the work is reading the other operand once from HBM
// (shapes of python/test/regression/test_performance.py:36-44; kernel contract of
// python/tutorials/03-matrix-multiplication.py:241-316).
//
// Written for out[s][l] = sum_k X[s][k] * Y[l][k]: X the small operand (S <= 64 rows), Y the
// streamed one (L rows).  The host maps (A, B) or (B^T, A^T) onto (X, Y).
//   * one workgroup per 32 rows of Y, its waves split K into contiguous ranges and meet in LDS at
//     the end - no tile reuse to organise, what matters is bytes in flight: every wave keeps
//     NS - 1 stages of 32 k (2 KiB of Y) outstanding;
//   * Y with K contiguous: each lane streams its own row straight into MFMA operand registers;
//   * Y with L contiguous (a row-major B): stages go global -> LDS by direct loads into a ring
//     private to the wave (no barriers in the loop) and come back transposed (ds_read_b64_tr_b16);
//   * X is re-read by every workgroup from L2, prefetched with the same depth through the same
//     ring: read back row-wise when K is contiguous, transposed when S is (the row-major B of a
//     product with N = 32 or 64).
#include "common.h"
#include "launch.h"
#include "formats.h"

namespace mi355 {

// Element families.  A stage is 64 BYTES of every operand row: 32 k of a 16-bit type (two
// 32x32x16 MFMAs, lane-group g feeding bytes 32 ks + 16 g .. + 16) or 64 k of fp8 (one 32x32x64
// MFMA, lane-group g feeding bytes 32 g .. + 32 as two 16-byte pieces).
template <typename V8_> struct Skinny16 { using V = V8_; static constexpr bool kF8 = false; static constexpr int kFmt = 0; };
template <int FMT> struct Skinny8 { using V = i32x4; static constexpr bool kF8 = true; static constexpr int kFmt = FMT; };  // 0 e4m3fn, 1 e5m2

// YM: 0 = K-contiguous Y, every lane streams its own row straight into registers (32-byte pieces of 32 rows per
//         instruction; kept for comparison);
//     1 = L-contiguous Y through LDS with a transposed read;
//     2 = K-contiguous Y through LDS (64-byte pieces of 16 rows per instruction, as for X);
//     3 = K-contiguous Y through LDS in whole 128-byte lines (8 rows per instruction): two stages share a tile of
//         [32 l][128 bytes of k] in a ring of its own; the loads of rows 0-15 ride with the odd stage before the
//         pair, those of rows 16-31 with its even stage, so every stage still issues two Y loads (needs K bytes a
//         multiple of 128);
//     4 = L-contiguous Y in whole 128-byte lines: the workgroup owns 64 columns (two 32-column tiles per wave, eight
//         waves that split K eight ways), a stage is a [32 k][64 l] tile fetched 8 k rows per instruction and read back
//         transposed (needs L a multiple of 64; chosen where L / 64 workgroups still cover the compute units)
template <typename E, int YM, int XM, int ST, int NW, int NS>
__global__ __launch_bounds__(NW * 64) void gemm_skinny_kernel(SkinnyArgs p) {
  using V8 = typename E::V;  // one 16-byte register group of an operand
  constexpr bool F8 = E::kF8;
  constexpr bool Y_LDS = YM == 1;
  constexpr int LT = YM == 4 ? 2 : 1;   // 32-column tiles of the output per wave
  constexpr int TT = LT * ST;           // accumulator tiles per wave: [LT][ST]
  static_assert(!F8 || (!Y_LDS && YM != 4 && XM == 2), "fp8: both operands K-contiguous, X through LDS");
  static_assert(XM != 3 || (NS % 2 == 0 && YM != 4), "pair tiles: a stage's parity is its slot's");
  constexpr int PD = NS - 1;          // stages in flight
  constexpr int LPS = (YM == 4 ? 4 : 2) + 2 * ST;   // vector-memory operations per stage: 2 (4) of Y, 2 per 32 rows of X
  // X: 0 = K contiguous, straight into registers (32-byte pieces of 32 rows per instruction: slower,
  //        kept for comparison); 1 = S contiguous, through LDS with a transposed read;
  //    2 = K contiguous, through LDS (64-byte pieces of 16 rows per instruction);
  //    3 = K contiguous, through LDS in whole 128-byte lines (8 rows per instruction): pair tiles of [32 ST s][128
  //        bytes of k] in a ring of their own, loaded like the pair tiles of YM 3 - first half of the rows with the odd
  //        stage before the pair, second half with its even stage (needs K bytes a multiple of 128; not for fp8)
  constexpr bool X_LDS = XM != 0;
  static_assert(!((Y_LDS || YM == 4) && XM == 1), "one operand at most is transposed through LDS");
  constexpr int XROW = 64 * ST;       // bytes of one k row of an S-contiguous X tile: S = 32 ST
  constexpr int YSLOT = (YM == 1 || YM == 2) ? 2048 : YM == 4 ? 4096 : 0;   // [32 k][32 l] 16-bit, [32 l][64 bytes of k], or [32 k][64 l]
  constexpr int ND = 4, YPAIR = 4096;            // YM == 3: ring of ND tiles [32 l][128 bytes of k] behind the stage ring
  constexpr int XSLOT = (XM == 1 || XM == 2) ? 2048 * ST : 0;   // [32 k][32 ST s] or [32 ST s][32 k]
  constexpr int XPAIR = 4096 * ST;               // XM == 3: [32 ST s][128 bytes of k]
  constexpr int XND = (YM == 3 && ST == 2) ? 3 : 4;   // pair tiles of X in its ring (three where four do not fit next to Y's; a tile is dead
                                                     // before the loads that re-use its place are issued from three on)
  constexpr int SLOT = YSLOT + XSLOT;            // bytes of one stage in LDS
  static_assert(PD * LPS < 64, "vmcnt has 6 bits");
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  LDS_PTR(char) const lds = (LDS_PTR(char))smem;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, g = lane >> 5, i16 = lane & 15, q = lane >> 4;
  // neighbouring 32-column blocks (the two halves of a 128-byte line of an L-contiguous Y) on one XCD
  const int l0 = xcd_remap(blockIdx.x, gridDim.x) * (32 * LT);

  const int nstages = p.K / (F8 ? 64 : 32);
  const int per = (YM == 3 || XM == 3) ? (((nstages + NW - 1) / NW + 1) & ~1) : (nstages + NW - 1) / NW;   // (pair tiles: whole pairs of stages)
  const int j_lo = wave * per, j_hi = min(nstages, j_lo + per);

  f32x16 acc[TT];
#pragma unroll
  for (int t = 0; t < TT; t++)
#pragma unroll
    for (int r = 0; r < 16; r++) acc[t][r] = 0.f;

  // Every load is a wave-uniform base (advancing with the stage) plus a fixed 32-bit lane offset.
  // lane (row l32, half g) feeds k = 16 ks + 8 g .. + 8 of MFMA sub-step ks
  unsigned xoff[ST];
#pragma unroll
  for (int t = 0; t < ST; t++) xoff[t] = (unsigned)min(32 * t + l32, p.S - 1) * (unsigned)p.x_pitch + g * 16;
  // S-contiguous X (x_pitch between k rows): direct load i of a stage moves k rows (16 / ST) i .. of XROW bytes
  const unsigned xdma = (unsigned)(lane / (4 * ST)) * (unsigned)p.x_pitch + (lane % (4 * ST)) * 16;
  // K-contiguous X through LDS: direct load i moves rows 16 i .. 16 i + 15, 64 bytes of k each; the
  // 16-byte chunk c of row r sits at position c ^ ((r >> 2) & 3) so that row-wise reads spread over the banks
  unsigned xdma2[2 * ST];
#pragma unroll
  for (int i = 0; i < 2 * ST; i++) {
    const int r = 16 * i + (lane >> 2);
    xdma2[i] = (unsigned)min(r, p.S - 1) * (unsigned)p.x_pitch + (((lane & 3) ^ ((r >> 2) & 3)) << 4);
  }
  // K-contiguous Y: the lane's own row
  const char* const ybase = (Y_LDS || YM == 4) ? p.Y + (int64_t)l0 * 2 : p.Y + (int64_t)l0 * p.y_pitch;
  // L-contiguous Y: direct load i of a stage moves k rows 16 i .. 16 i + 15, 64 bytes (32 l) each
  const unsigned yoff = Y_LDS ? (unsigned)(lane >> 2) * (unsigned)p.y_pitch + (lane & 3) * 16
                              : (unsigned)l32 * (unsigned)p.y_pitch + g * (F8 ? 32 : 16);
  const unsigned ring = lds_addr(lds) + wave * (NS * SLOT);
  // transposed read: 16 lanes fetch 4 k rows x 16 l and receive 4 k values of one l each;
  // lane -> k row 8 g + i16 / 4 (+ 4 for the second read), l = 16 (q & 1) + i16
  const unsigned tl = ring + (8 * (q >> 1) + (i16 >> 2)) * (XM == 1 ? XROW : 64) + (q & 1) * 32 + (i16 & 3) * 8;
  // row-wise read of the K-contiguous X tile: row s = 32 t + l32, chunk (2 ks + g) ^ ((s >> 2) & 3)
  // (fp8: the two pieces of the lane's 32 bytes, chunks 2 g and 2 g + 1)
  unsigned xrd[2];
#pragma unroll
  for (int ks = 0; ks < 2; ks++) xrd[ks] = ring + YSLOT + l32 * 64 + ((((F8 ? 2 * g + ks : 2 * ks + g)) ^ ((l32 >> 2) & 3)) << 4);

  // K-contiguous Y through LDS: direct load i moves rows 16 i .. 16 i + 15, 64 bytes of k each, chunk c of row r at
  // position c ^ ((r >> 2) & 3); read back row-wise like X
  unsigned ydma2[2], yrd[2];
#pragma unroll
  for (int i = 0; i < 2; i++) {
    const int r = 16 * i + (lane >> 2);
    ydma2[i] = (unsigned)r * (unsigned)p.y_pitch + (((lane & 3) ^ ((r >> 2) & 3)) << 4);
  }
#pragma unroll
  for (int ks = 0; ks < 2; ks++) yrd[ks] = ring + l32 * 64 + ((((F8 ? 2 * g + ks : 2 * ks + g)) ^ ((l32 >> 2) & 3)) << 4);
  // YM == 3: load instruction i of a pair moves rows 8 i .. 8 i + 7, all 128 bytes; chunk c of row r at position
  // c ^ ((r >> 1) & 7) (rows are 128 bytes apart: two rows per sweep of the banks)
  const unsigned yring = lds_addr(lds) + NW * (NS * SLOT) + wave * (ND * YPAIR);
  // (row r = 8 i + lane / 8: (r >> 1) & 7 = 4 (i & 1) + lane / 16; the lane's slot is lane % 8, so it fetches chunk
  // (lane % 8) ^ that term)
  unsigned ydma3[2];
#pragma unroll
  for (int i = 0; i < 2; i++) ydma3[i] = (unsigned)(lane >> 3) * (unsigned)p.y_pitch + (((lane & 7) ^ (4 * i + (lane >> 4))) << 4);
  unsigned yrd3[2];
#pragma unroll
  for (int ks = 0; ks < 2; ks++) yrd3[ks] = yring + l32 * 128 + ((((F8 ? 2 * g + ks : 2 * ks + g)) ^ ((l32 >> 1) & 7)) << 4);
  // XM == 3: the same for X; instruction i of a pair (0 .. 4 ST - 1) moves rows 8 i .. 8 i + 7 (rows beyond S fetch
  // row S - 1 into their place)
  const unsigned xring = lds_addr(lds) + NW * (NS * SLOT) + (YM == 3 ? NW * (ND * YPAIR) : 0) + wave * (XND * XPAIR);
  unsigned xdma3[XM == 3 ? 4 * ST : 1];
  unsigned xrd3[2];
  if constexpr (XM == 3) {
#pragma unroll
    for (int i = 0; i < 4 * ST; i++)
      xdma3[i] = (unsigned)min(8 * i + (lane >> 3), p.S - 1) * (unsigned)p.x_pitch + (((lane & 7) ^ (4 * (i & 1) + (lane >> 4))) << 4);
#pragma unroll
    for (int ks = 0; ks < 2; ks++) xrd3[ks] = xring + l32 * 128 + (((2 * ks + g) ^ ((l32 >> 1) & 7)) << 4);
  }
  // YM == 4: load instruction i of a stage moves k rows 8 i .. 8 i + 7 of 128 bytes (64 l); in the rows with bit 1 of
  // k set the two 64-byte halves change places (chunk c at position c ^ 4), so that the four k rows of a transposed
  // read - 128 bytes apart - lie in four different quarters of the banks.  Lane of a read: k row 8 g + i16 / 4 (+ 4,
  // 16, 20 by the instruction offset: bit 1 of k stays), columns 16 (q & 1) + 4 (i16 & 3) .. of tile lt.
  const unsigned yoff4 = (unsigned)(lane >> 3) * (unsigned)p.y_pitch + (((lane & 7) ^ (((lane >> 4) & 1) << 2)) << 4);
  const unsigned tl4 = ring + (8 * (q >> 1) + (i16 >> 2)) * 128 + (((2 * (q & 1) + ((i16 & 3) >> 1)) ^ (((i16 >> 3) & 1) << 2)) << 4) + (i16 & 1) * 8;
  V8 xr[NS][2][ST], yr[NS][2];
  auto issue = [&](int j, auto SLOT_) {
    constexpr int sl = decltype(SLOT_)::value;
    if constexpr (Y_LDS) {
      const char* src = ybase + (int64_t)j * 32 * p.y_pitch;
      async_copy16_sbase(src, yoff, ring + sl * SLOT);
      async_copy16_sbase(src + 16 * p.y_pitch, yoff, ring + sl * SLOT + 1024);
    } else if constexpr (YM == 4) {
      const char* src = ybase + (int64_t)j * 32 * p.y_pitch;
#pragma unroll
      for (int i = 0; i < 4; i++) async_copy16_sbase(src + (int64_t)(8 * i) * p.y_pitch, yoff4, ring + sl * SLOT + i * 1024);
    } else if constexpr (YM == 2) {
      const char* src = ybase + (int64_t)j * 64;
      async_copy16_sbase(src, ydma2[0], ring + sl * SLOT);
      async_copy16_sbase(src, ydma2[1], ring + sl * SLOT + 1024);
    } else if constexpr (YM == 3) {
      // odd stage: rows 0-15 of the NEXT pair (the last pair again where there is none); even stage: rows 16-31 of its own
      const int d = min((j + 1) >> 1, (j_hi >> 1) - 1), half = (j & 1) ^ 1;
      const char* src = ybase + (int64_t)d * 128 + (int64_t)(16 * half) * p.y_pitch;
      const unsigned dst = yring + (d & (ND - 1)) * YPAIR + half * 2048;
      // (the XOR term of rows 8 .. 15 of a half is 4 more than that of rows 0 .. 7)
      async_copy16_sbase(src, ydma3[0], dst);
      async_copy16_sbase(src + 8 * p.y_pitch, ydma3[1], dst + 1024);
    } else {
      const char* src = ybase + (int64_t)j * 64;
      load16_sbase<0>(yr[sl][0], src, yoff);
      load16_sbase<(F8 ? 16 : 32)>(yr[sl][1], src, yoff);
    }
    if constexpr (XM == 1) {
      const char* xsrc = p.X + (int64_t)j * 32 * p.x_pitch;
#pragma unroll
      for (int i = 0; i < 2 * ST; i++)
        async_copy16_sbase(xsrc + (int64_t)i * (16 / ST) * p.x_pitch, xdma, ring + sl * SLOT + YSLOT + i * 1024);
    } else if constexpr (XM == 3) {
      // odd stage: first half of the rows of the NEXT pair (the last pair again where there is none); even: second half of its own
      const int d = min((j + 1) >> 1, (j_hi >> 1) - 1), half = (j & 1) ^ 1;
      const char* xsrc = p.X + (int64_t)d * 128;
      const unsigned dst = xring + (d % XND) * XPAIR + half * (2 * ST * 1024);
      static_for<2 * ST>([&](auto I_) {
        constexpr int i = decltype(I_)::value;
        if (half) async_copy16_sbase(xsrc, xdma3[2 * ST + i], dst + i * 1024);
        else async_copy16_sbase(xsrc, xdma3[i], dst + i * 1024);
      });
    } else if constexpr (XM == 2) {
      const char* xsrc = p.X + (int64_t)j * 64;
#pragma unroll
      for (int i = 0; i < 2 * ST; i++) async_copy16_sbase(xsrc, xdma2[i], ring + sl * SLOT + YSLOT + i * 1024);
    } else {
      const char* xsrc = p.X + (int64_t)j * 64;
#pragma unroll
      for (int t = 0; t < ST; t++) {
        load16_sbase<0>(xr[sl][0][t], xsrc, xoff[t]);
        load16_sbase<32>(xr[sl][1][t], xsrc, xoff[t]);
      }
    }
  };
  auto compute = [&](const int j, auto SLOT_) {
    constexpr int sl = decltype(SLOT_)::value;
    V8 yfl[LT][2];
    V8 (&yf)[2] = yfl[0];
    if constexpr (YM == 4) {
      i32x2 lo[2][2], hi[2][2];
      static_for<2>([&](auto LT_) {
        constexpr int lt = decltype(LT_)::value;
        const unsigned ad = tl4 ^ (lt * 64u);   // (the second tile's chunks are 4 further: bit 2 of the position)
        lo[lt][0] = lds_read_tr16_b64<sl * SLOT>(ad);
        hi[lt][0] = lds_read_tr16_b64<sl * SLOT + 4 * 128>(ad);
        lo[lt][1] = lds_read_tr16_b64<sl * SLOT + 16 * 128>(ad);
        hi[lt][1] = lds_read_tr16_b64<sl * SLOT + 20 * 128>(ad);
      });
      lds_wait<0>();
#pragma unroll
      for (int lt = 0; lt < 2; lt++)
#pragma unroll
        for (int ks = 0; ks < 2; ks++) {
          lds_use(lo[lt][ks]);
          lds_use(hi[lt][ks]);
          yfl[lt][ks] = __builtin_bit_cast(V8, (i32x4)__builtin_shufflevector(lo[lt][ks], hi[lt][ks], 0, 1, 2, 3));
        }
    } else if constexpr (Y_LDS) {
      i32x2 lo[2], hi[2];
      lo[0] = lds_read_tr16_b64<sl * SLOT>(tl);
      hi[0] = lds_read_tr16_b64<sl * SLOT + 4 * 64>(tl);
      lo[1] = lds_read_tr16_b64<sl * SLOT + 16 * 64>(tl);
      hi[1] = lds_read_tr16_b64<sl * SLOT + 20 * 64>(tl);
      lds_wait<0>();
#pragma unroll
      for (int ks = 0; ks < 2; ks++) {
        lds_use(lo[ks]);
        lds_use(hi[ks]);
        yf[ks] = __builtin_bit_cast(V8, (i32x4)__builtin_shufflevector(lo[ks], hi[ks], 0, 1, 2, 3));
      }
    } else if constexpr (YM == 3) {
      // (the stage's parity is the slot's: ranges start on even stages and the ring has an even number of slots;
      // the odd stage's chunks are 4 further, which flips bit 2 of the swizzled position)
      const unsigned yb = (unsigned)((j >> 1) & (ND - 1)) * YPAIR;
      i32x4 yv[2];
      yv[0] = lds_read_b128<0>((yrd3[0] ^ ((sl & 1) * 64u)) + yb);
      yv[1] = lds_read_b128<0>((yrd3[1] ^ ((sl & 1) * 64u)) + yb);
      lds_wait<0>();
      lds_use(yv[0]);
      lds_use(yv[1]);
      yf[0] = __builtin_bit_cast(V8, yv[0]);
      yf[1] = __builtin_bit_cast(V8, yv[1]);
    } else if constexpr (YM == 2) {
      i32x4 yv[2];
      yv[0] = lds_read_b128<sl * SLOT>(yrd[0]);
      yv[1] = lds_read_b128<sl * SLOT>(yrd[1]);
      lds_wait<0>();
      lds_use(yv[0]);
      lds_use(yv[1]);
      yf[0] = __builtin_bit_cast(V8, yv[0]);
      yf[1] = __builtin_bit_cast(V8, yv[1]);
    } else {
      lds_use(yr[sl][0]);
      lds_use(yr[sl][1]);
      yf[0] = yr[sl][0];
      yf[1] = yr[sl][1];
    }
    V8 xf[2][ST];
    if constexpr (XM == 3) {
      const unsigned xb = (unsigned)((j >> 1) % XND) * XPAIR;
      i32x4 xv[2][ST];
      static_for<2>([&](auto KS_) {
        constexpr int ks = decltype(KS_)::value;
        static_for<ST>([&](auto T_) {
          constexpr int t = decltype(T_)::value;
          xv[ks][t] = lds_read_b128<t * 4096>((xrd3[ks] ^ ((sl & 1) * 64u)) + xb);
        });
      });
      lds_wait<0>();
#pragma unroll
      for (int ks = 0; ks < 2; ks++)
#pragma unroll
        for (int t = 0; t < ST; t++) {
          lds_use(xv[ks][t]);
          xf[ks][t] = __builtin_bit_cast(V8, xv[ks][t]);
        }
    } else if constexpr (XM == 2) {
      i32x4 xv[2][ST];
      static_for<2>([&](auto KS_) {
        constexpr int ks = decltype(KS_)::value;
        static_for<ST>([&](auto T_) {
          constexpr int t = decltype(T_)::value;
          xv[ks][t] = lds_read_b128<sl * SLOT + t * 2048>(xrd[ks]);
        });
      });
      lds_wait<0>();
#pragma unroll
      for (int ks = 0; ks < 2; ks++)
#pragma unroll
        for (int t = 0; t < ST; t++) {
          lds_use(xv[ks][t]);
          xf[ks][t] = __builtin_bit_cast(V8, xv[ks][t]);
        }
    } else if constexpr (XM == 1) {
      i32x2 lo[2][ST], hi[2][ST];
      static_for<2>([&](auto KS_) {
        constexpr int ks = decltype(KS_)::value;
        static_for<ST>([&](auto T_) {
          constexpr int t = decltype(T_)::value;
          lo[ks][t] = lds_read_tr16_b64<sl * SLOT + YSLOT + 16 * ks * XROW + t * 64>(tl);
          hi[ks][t] = lds_read_tr16_b64<sl * SLOT + YSLOT + (16 * ks + 4) * XROW + t * 64>(tl);
        });
      });
      lds_wait<0>();
#pragma unroll
      for (int ks = 0; ks < 2; ks++)
#pragma unroll
        for (int t = 0; t < ST; t++) {
          lds_use(lo[ks][t]);
          lds_use(hi[ks][t]);
          xf[ks][t] = __builtin_bit_cast(V8, (i32x4)__builtin_shufflevector(lo[ks][t], hi[ks][t], 0, 1, 2, 3));
        }
    } else {
#pragma unroll
      for (int ks = 0; ks < 2; ks++)
#pragma unroll
        for (int t = 0; t < ST; t++) {
          lds_use(xr[sl][ks][t]);
          xf[ks][t] = xr[sl][ks][t];
        }
    }
    if constexpr (F8) {
#pragma unroll
      for (int t = 0; t < ST; t++) {
        const i32x8 a = __builtin_shufflevector(yf[0], yf[1], 0, 1, 2, 3, 4, 5, 6, 7);
        const i32x8 b = __builtin_shufflevector(xf[0][t], xf[1][t], 0, 1, 2, 3, 4, 5, 6, 7);
#if MI355_DEVICE_PASS
        acc[t] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, acc[t], E::kFmt, E::kFmt, 0, 0, 0, 0);
#endif
      }
    } else {
#pragma unroll
      for (int ks = 0; ks < 2; ks++)
#pragma unroll
        for (int lt = 0; lt < LT; lt++)
#pragma unroll
          for (int t = 0; t < ST; t++) acc[lt * ST + t] = mfma32(yfl[lt][ks], xf[ks][t], acc[lt * ST + t]);
    }
  };

  if (j_lo < j_hi) {
    // past the end of the range the last stage is fetched again: the number of outstanding
    // operations, and with it the partial wait, stays uniform
    if constexpr (YM == 3) {
      // rows 0-15 of the first pair (in the stream they ride with the odd stage before a pair)
      const int d = j_lo >> 1;
      const char* src = ybase + (int64_t)d * 128;
      const unsigned dst = yring + (d & (ND - 1)) * YPAIR;
      async_copy16_sbase(src, ydma3[0], dst);
      async_copy16_sbase(src + 8 * p.y_pitch, ydma3[1], dst + 1024);
    }
    if constexpr (XM == 3) {
      // first half of the rows of the first pair
      const int d = j_lo >> 1;
      const char* xsrc = p.X + (int64_t)d * 128;
      const unsigned dst = xring + (d % XND) * XPAIR;
      static_for<2 * ST>([&](auto I_) { async_copy16_sbase(xsrc, xdma3[decltype(I_)::value], dst + decltype(I_)::value * 1024); });
    }
    static_for<PD>([&](auto S_) { issue(min(j_lo + decltype(S_)::value, j_hi - 1), S_); });
    for (int j = j_lo; j < j_hi; j += NS) {
      static_for<NS>([&](auto U_) {
        constexpr int u = decltype(U_)::value;
        if (j + u < j_hi) {
          issue(min(j + u + PD, j_hi - 1), std::integral_constant<int, (u + PD) % NS>{});
          wait_vmcnt<PD * LPS>();
          __builtin_amdgcn_sched_barrier(0);
          compute(j + u, U_);
          __builtin_amdgcn_sched_barrier(0);
        }
      });
    }
    wait_vmcnt<0>();
  }

  // ---- sum the waves' partial tiles through LDS (the rings are dead after the barrier)
  __syncthreads();
  LDS_PTR(float) const red = (LDS_PTR(float))lds;  // [NW][TT * 16][64]
#pragma unroll
  for (int t = 0; t < TT; t++)
#pragma unroll
    for (int r = 0; r < 16; r++) red[(wave * TT * 16 + t * 16 + r) * 64 + lane] = acc[t][r];
  __syncthreads();
  float alpha = 1.f;
  if (p.a_scale) alpha *= *p.a_scale;
  if (p.b_scale) alpha *= *p.b_scale;
  constexpr int RPW = TT * 16 / NW;  // accumulator registers finished by each wave
  static_assert(RPW >= 1, "more waves than accumulator registers");
#pragma unroll
  for (int e = 0; e < RPW; e++) {
    const int rr = wave * RPW + e, tt = rr >> 4, r = rr & 15, lt = tt / ST, t = tt % ST;
    float v = 0.f;
#pragma unroll
    for (int w = 0; w < NW; w++) v += red[(w * TT * 16 + rr) * 64 + lane];
    v *= alpha;
    // register r of lane: row l = 8 (r / 4) + 4 g + r % 4 of the tile, column s = l32
    const int s = 32 * t + l32, l = l0 + 32 * lt + (r >> 2) * 8 + g * 4 + (r & 3);
    if (s < p.S && l < p.L) {
      if (p.aux) v += load_aux(p.aux, (int64_t)s * p.aux_ss + (int64_t)l * p.aux_sl, p.aux_dtype);
      if (p.activation == 1) v = v >= 0.f ? v : 0.01f * v;
      const int64_t off = (int64_t)s * p.cs + (int64_t)l * p.cl;
      if (p.out_dtype == 4) ((float*)p.C)[off] = v;
      else if (p.out_dtype == 2) ((uint8_t*)p.C)[off] = f32_to_e4m3(v);
      else if (p.out_dtype == 3) ((uint8_t*)p.C)[off] = f32_to_e5m2(v);
      else if (p.out_dtype == 1) ((__bf16*)p.C)[off] = (__bf16)v;
      else ((_Float16*)p.C)[off] = (_Float16)v;
    }
  }
}

template <typename E, int YM, int XM, int ST>
static int launch_skinny(const SkinnyArgs& p, hipStream_t stream) {
  // four waves with three stages in flight each already saturate what this access pattern gets
  // from HBM; the small LDS footprint lets several workgroups share a CU
  // (YM 4, 64 columns per workgroup: half as many workgroups, so eight waves each split K eight ways)
  constexpr int NW = YM == 4 ? 8 : 4, NS = YM == 4 ? 3 : 4;
  constexpr int LT = YM == 4 ? 2 : 1;
  constexpr int ring = NW * NS * ((YM == 1 || YM == 2 ? 2048 : YM == 4 ? 4096 : 0) + (XM == 1 || XM == 2 ? 2048 * ST : 0)) + (YM == 3 ? NW * 4 * 4096 : 0) +
                       (XM == 3 ? NW * ((YM == 3 && ST == 2) ? 3 : 4) * 4096 * ST : 0), red = NW * LT * ST * 16 * 64 * 4;
  static_assert(ring <= 160 * 1024, "LDS of one CU");
  constexpr int smem = ring > red ? ring : red;
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)gemm_skinny_kernel<E, YM, XM, ST, NW, NS>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) return (int)e;
    attr_set = true;
  }
  gemm_skinny_kernel<E, YM, XM, ST, NW, NS><<<dim3(p.L / (32 * LT)), dim3(NW * 64), smem, stream>>>(p);
  return (int)hipGetLastError();
}

// S <= 64, whole 32-row blocks of Y and whole 64-byte stages; pitches in bytes, 16-byte aligned rows,
// small enough that 64 rows of X / 32 rows of Y are reached with 32-bit offsets.  An S-contiguous
// X (x_kmajor false) needs S = 32 or 64 and a K-contiguous Y.  elem_bytes = 2 or 1 (fp8: both
// operands K-contiguous).
bool gemm_skinny_ok(const SkinnyArgs& p, bool y_kmajor, bool x_kmajor, int elem_bytes) {
  if (!x_kmajor && (!y_kmajor || (p.S != 32 && p.S != 64))) return false;
  if (elem_bytes == 1 && !(x_kmajor && y_kmajor)) return false;
  const int64_t kb = (int64_t)p.K * elem_bytes;
  return p.S >= 1 && p.S <= 64 && p.L >= 32 && p.L % 32 == 0 && kb >= 64 && kb % 64 == 0 &&
         p.x_pitch % 16 == 0 && p.y_pitch % 16 == 0 && p.x_pitch < (1 << 25) && p.y_pitch < (1 << 26);
}

// how a K-contiguous Y travels (see YM above)
#ifndef MI355_SKINNY_Y_KMAJOR_MODE
#define MI355_SKINNY_Y_KMAJOR_MODE 3
#endif
constexpr int YK = MI355_SKINNY_Y_KMAJOR_MODE;
#ifndef MI355_SKINNY_Y_LMAJOR_MODE
#define MI355_SKINNY_Y_LMAJOR_MODE 4
#endif
// a K-contiguous Y: whole lines (mode 3) where K bytes are a multiple of 128, else 64-byte pieces
// how the 33 .. 64 K-contiguous rows of X travel next to an L-contiguous Y where K bytes are a multiple of 128 (see XM in
// the kernel): 3 = whole lines (64 x 8192 x 8192 3520 -> 3745 GB/s), 2 = 64-byte pieces.  With at most 32 rows, and
// next to a K-contiguous Y in pair tiles of its own, whole lines for X measured +-0 and -1.2 %: 64-byte pieces there.
#ifndef MI355_SKINNY_X_KMAJOR_MODE
#define MI355_SKINNY_X_KMAJOR_MODE 3
#endif
template <typename E, int XM, int ST>
static int launch_skinny_yk(const SkinnyArgs& p, int elem_bytes, hipStream_t stream) {
  if constexpr (YK == 3) {
    if (((int64_t)p.K * elem_bytes) % 128 == 0) {
      // (49 .. 64 K-contiguous rows of X: whole lines for X too, in a ring of three pair tiles next to Y's four; 16-bit.
      // 64 x 8192 x 8192 with a K-contiguous weight 32.0 -> 30.0 us, 8192 x 64 x 8192 30.1 -> 28.2; but 48 rows 26.0 -> 27.5)
      if constexpr (MI355_SKINNY_X_KMAJOR_MODE == 3 && XM == 2 && ST == 2 && !E::kF8) {
        if (p.S > 48) return launch_skinny<E, 3, 3, ST>(p, stream);
      }
      return launch_skinny<E, 3, XM, ST>(p, stream);
    }
    return launch_skinny<E, 2, XM, ST>(p, stream);
  } else {
    return launch_skinny<E, YK, XM, ST>(p, stream);
  }
}

template <typename V8>
static int launch_skinny_v(const SkinnyArgs& p, bool y_kmajor, bool x_kmajor, hipStream_t stream) {
  using E = Skinny16<V8>;
  const bool two = p.S > 32;
  if (!x_kmajor) return two ? launch_skinny_yk<E, 1, 2>(p, 2, stream) : launch_skinny_yk<E, 1, 1>(p, 2, stream);
  if (y_kmajor) return two ? launch_skinny_yk<E, 2, 2>(p, 2, stream) : launch_skinny_yk<E, 2, 1>(p, 2, stream);
  // an L-contiguous Y: whole lines (64 columns per workgroup) where L is a multiple of 64
  // (at most 32 rows of X: eight waves of two column tiles each fit LDS; and enough columns that 64 per workgroup still
  // give every compute unit one - 16 x 16384 x 8192 5250 -> 6050 GB/s, but 16 x 8192 x 8192, 128 workgroups, 4685 -> 4580)
  if (MI355_SKINNY_Y_LMAJOR_MODE == 4 && p.L % 64 == 0 && !two && p.cus > 0 && p.L / 64 >= p.cus) return launch_skinny<E, 4, 2, 1>(p, stream);
  if (MI355_SKINNY_X_KMAJOR_MODE == 3 && two && ((int64_t)p.K * 2) % 128 == 0) return launch_skinny<E, 1, 3, 2>(p, stream);
  return two ? launch_skinny<E, 1, 2, 2>(p, stream) : launch_skinny<E, 1, 2, 1>(p, stream);
}

// kind: 0 fp16, 1 bf16, 2 fp8 e4m3fn, 3 fp8 e5m2 (the dtype codes of the C ABI)
int gemm_skinny_launch(const SkinnyArgs& p, int kind, bool y_kmajor, bool x_kmajor, hipStream_t stream) {
  const bool two = p.S > 32;
  if (kind == 2) return two ? launch_skinny_yk<Skinny8<0>, 2, 2>(p, 1, stream) : launch_skinny_yk<Skinny8<0>, 2, 1>(p, 1, stream);
  if (kind == 3) return two ? launch_skinny_yk<Skinny8<1>, 2, 2>(p, 1, stream) : launch_skinny_yk<Skinny8<1>, 2, 1>(p, 1, stream);
  return kind == 1 ? launch_skinny_v<bf16x8>(p, y_kmajor, x_kmajor, stream) : launch_skinny_v<f16x8>(p, y_kmajor, x_kmajor, stream);
}

}  // namespace mi355

// fp16 / bf16 tiled GEMM for gfx950: C[M,N] = act(alpha * A[M,K] @ B[K,N]), fp32 accumulate.
//
// The device-side counterpart of the reference `matmul_kernel`
// (python/tutorials/03-matrix-multiplication.py:241-316): one workgroup per BM x BN tile of C,
// grouped tile order (:265-273), K loop in BK = 64 steps (:294-303), epilogue activation and
// cast (:304-316).  Built MI355X-first instead of translated:
//   * operands go global -> LDS with direct 16-byte loads into two LDS stages (no register
//     staging); the tile for step k+1 is in flight while step k is multiplied;
//   * LDS rows are XOR-swizzled so that ds_read_b128 / ds_read_b64_tr_b16 are conflict free;
//   * a row-major B[K,N] is transposed on the fly by the LDS transpose read, a K-major B
//     (the `b.T` view the reference passes for fp8, :378-382) uses plain 128-bit reads;
//   * 32x32x16 MFMA, operands swapped so every lane owns 4 consecutive columns of one C row
//     and stores 8 bytes at a time;
//   * workgroup ids are remapped per XCD before the grouped ordering.
#include "common.h"
#include "launch.h"

namespace mi355 {

template <typename T> struct Vec;
template <> struct Vec<__bf16> { using v8 = bf16x8; using v4 = bf16x4; };
template <> struct Vec<_Float16> { using v8 = f16x8; using v4 = f16x4; };

// Source pointers / guarded copy for a row-major [64 x BN] tile of B (rows are k, BN*2 bytes each).
// 32-byte groups of a row are XORed with (k & 3): the transpose read of one 16-lane group touches
// 4 consecutive k rows x 32 bytes, which then fall into 4 different bank groups.
template <int BN, int NW>
struct TileCopyKN {
  static constexpr int kChunksPerRow = BN / 8;            // 16-byte chunks per k row
  static constexpr int kRowsPerInst = 64 / kChunksPerRow; // k rows moved by one wave instruction
  static constexpr int kIters = 64 / kRowsPerInst / NW;
  static_assert(kRowsPerInst >= 1 && kIters >= 1, "tile too small for this wave count");

  __device__ static int row(int wave, int lane, int i) { return (i * NW + wave) * kRowsPerInst + lane / kChunksPerRow; }
  __device__ static int col16(int lane, int r) {  // logical 16-byte chunk this lane fetches
    int pc16 = lane % kChunksPerRow;
    int lc32 = (pc16 >> 1) ^ (r & 3);
    return lc32 * 2 + (pc16 & 1);
  }
};

template <typename T, int BM, int BN, int WM, int WN, bool B_KMAJOR>
__global__ __launch_bounds__(WM * WN * 64, 1) void gemm16_kernel(GemmArgs p) {
  using V8 = typename Vec<T>::v8;
  using V4 = typename Vec<T>::v4;
  constexpr int NW = WM * WN, TM = BM / WM, TN = BN / WN, MT = TM / 32, NT = TN / 32;
  constexpr int A_BYTES = BM * 128, B_BYTES = BN * 128, STAGE = A_BYTES + B_BYTES;
  using CopyA = TileCopy128<BM, NW>;
  using CopyBk = TileCopy128<BN, NW>;
  using CopyBn = TileCopyKN<BN, NW>;
  constexpr int ITB = B_KMAJOR ? CopyBk::kIters : CopyBn::kIters;

  // Two LDS stages of STAGE bytes each (dynamic LDS: 2 * STAGE bytes at launch).
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  LDS_PTR(char) const lds0 = (LDS_PTR(char))smem;
  LDS_PTR(char) const lds1 = lds0 + STAGE;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WN, wn = wave % WN;

  const int num_m = (p.M + BM - 1) / BM, num_n = (p.N + BN - 1) / BN;
  int pid = xcd_remap(blockIdx.x, num_m * num_n);
  int pm, pn;
  grouped_tile(pid, num_m, num_n, p.group_m, pm, pn);
  const int m0 = pm * BM, n0 = pn * BN;

  // per-lane global source pointers of the k = 0 tile
  const char* srcA[CopyA::kIters];
  const char* srcB[ITB];
#pragma unroll
  for (int i = 0; i < CopyA::kIters; i++) srcA[i] = CopyA::src(p.A, p.lda, m0, p.M, wave, lane, i);
#pragma unroll
  for (int i = 0; i < ITB; i++) {
    if constexpr (B_KMAJOR) {
      srcB[i] = CopyBk::src(p.B, p.ldb, n0, p.N, wave, lane, i);
    } else {
      int r = CopyBn::row(wave, lane, i);
      int n = n0 + CopyBn::col16(lane, r) * 8;
      n = n < p.N ? n : p.N - 8;  // N % 8 == 0 on this path: clamp whole chunks
      srcB[i] = p.B + (int64_t)r * p.ldb + (int64_t)n * 2;
    }
  }
  const int64_t stepA = 128, stepB = B_KMAJOR ? (int64_t)128 : 64 * p.ldb;

  auto issue_tile = [&](int kt, LDS_PTR(char) a) {
    LDS_PTR(char) b = a + A_BYTES;
#pragma unroll
    for (int i = 0; i < CopyA::kIters; i++)
      async_copy16(srcA[i] + kt * stepA, (LDS_PTR(void))(a + (i * NW + wave) * 1024));
#pragma unroll
    for (int i = 0; i < ITB; i++)
      async_copy16(srcB[i] + kt * stepB, (LDS_PTR(void))(b + (i * NW + wave) * 1024));
  };
  // Last, partial K tile: chunks past K are written as zeros (the reference masks them to 0,
  // python/tutorials/03-matrix-multiplication.py:297-298); goes through registers.
  auto guarded_tile = [&](int kt, LDS_PTR(char) a) {
    LDS_PTR(char) b = a + A_BYTES;
    const int kbase = kt * 64;
#pragma unroll
    for (int i = 0; i < CopyA::kIters; i++) {
      int r = (i * NW + wave) * 8 + (lane >> 3);
      int k = kbase + (((lane & 7) ^ (r & 7)) << 3);
      i32x4 v = {0, 0, 0, 0};
      if (k < p.K) v = *(const i32x4*)(srcA[i] + kt * stepA);
      *(LDS_PTR(i32x4))(a + (i * NW + wave) * 1024 + lane * 16) = v;
    }
#pragma unroll
    for (int i = 0; i < ITB; i++) {
      int k;
      if constexpr (B_KMAJOR) {
        int r = (i * NW + wave) * 8 + (lane >> 3);
        k = kbase + (((lane & 7) ^ (r & 7)) << 3);
      } else {
        k = kbase + CopyBn::row(wave, lane, i);
      }
      i32x4 v = {0, 0, 0, 0};
      if (k < p.K) v = *(const i32x4*)(srcB[i] + kt * stepB);
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

  const int nfull = p.K / 64;

  // Per-lane LDS byte offsets of the MFMA fragments inside one stage.
  //   K-major operand (A always, B when B_KMAJOR): lane reads row (l%32), 16-byte chunk
  //   (2*ks + l/32), swizzled -> one offset per ks; 32-row sub-tiles add t * 4096.
  //   Row-major B: transpose read, lane i of a 16-lane group q addresses k row
  //   16*ks + 8*(q/2) + i/4 (+4 for the second half) and 32-byte group (n/16) ^ (k & 3).
  const int l32 = lane & 31, g = lane >> 5;
  const int i16 = lane & 15, q = lane >> 4;
  unsigned offA[4], offB[4];
#pragma unroll
  for (int ks = 0; ks < 4; ks++) {
    offA[ks] = swz128(wm * TM + l32, ks * 2 + g);
    if constexpr (B_KMAJOR) {
      offB[ks] = A_BYTES + swz128(wn * TN + l32, ks * 2 + g);
    }
  }
  if constexpr (!B_KMAJOR) {
    // offB[par]: sub-tiles t with parity par; k row without the ks / +4 terms
    int k = (q >> 1) * 8 + (i16 >> 2);
#pragma unroll
    for (int par = 0; par < 2; par++) {
      int c32 = (wn * TN + par * 32) / 16 + (q & 1);
      offB[par] = A_BYTES + k * (BN * 2) + ((c32 ^ (k & 3)) << 5) + (i16 & 3) * 8;
    }
  }

  struct Frags { V8 a[MT]; V8 b[NT]; };
  auto read_frags = [&](unsigned base, auto KS, Frags& f) {
    constexpr int ks = decltype(KS)::value;
    static_for<MT>([&](auto T_) {
      constexpr int t = decltype(T_)::value;
      f.a[t] = __builtin_bit_cast(V8, lds_read_b128<t * 4096>(base + offA[ks]));
    });
    static_for<NT>([&](auto T_) {
      constexpr int t = decltype(T_)::value;
      if constexpr (B_KMAJOR) {
        f.b[t] = __builtin_bit_cast(V8, lds_read_b128<t * 4096>(base + offB[ks]));
      } else {
        constexpr int imm = ks * 16 * BN * 2 + (t / 2) * 128;
        i32x2 lo = lds_read_tr16_b64<imm>(base + offB[t & 1]);
        i32x2 hi = lds_read_tr16_b64<imm + 4 * BN * 2>(base + offB[t & 1]);
        i32x4 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3);
        f.b[t] = __builtin_bit_cast(V8, both);
      }
    });
  };
  constexpr int kReadsPerStep = MT + NT * (B_KMAJOR ? 1 : 2);
  auto use_frags = [&](Frags& f) {
#pragma unroll
    for (int t = 0; t < MT; t++) lds_use(f.a[t]);
#pragma unroll
    for (int t = 0; t < NT; t++) lds_use(f.b[t]);
  };
  auto mma = [&](const Frags& f) {
#pragma unroll
    for (int i = 0; i < MT; i++)
#pragma unroll
      for (int j = 0; j < NT; j++) acc[i][j] = mfma32(f.b[j], f.a[i], acc[i][j]);  // D[n][m]
  };

  // One BK = 64 tile: fragments of sub-step ks+1 are requested before the MFMAs of sub-step ks.
  auto compute_tile = [&](LDS_PTR(char) stage) {
    const unsigned base = lds_addr(stage);
    Frags f0, f1;
    read_frags(base, std::integral_constant<int, 0>{}, f0);
    read_frags(base, std::integral_constant<int, 1>{}, f1);
    lds_wait<kReadsPerStep>(); use_frags(f0); mma(f0);
    read_frags(base, std::integral_constant<int, 2>{}, f0);
    lds_wait<kReadsPerStep>(); use_frags(f1); mma(f1);
    read_frags(base, std::integral_constant<int, 3>{}, f1);
    lds_wait<kReadsPerStep>(); use_frags(f0); mma(f0);
    lds_wait<0>(); use_frags(f1); mma(f1);
  };

  // K loop over the full tiles, two per trip so that each half names its LDS stage statically:
  // the tile for step kt+1 streams into the idle stage while step kt is multiplied out of the other.
  if (nfull > 0) {
    issue_tile(0, lds0);
    wait_all();
    __syncthreads();
    for (int kt = 0; kt < nfull; kt += 2) {
      if (kt + 1 < nfull) issue_tile(kt + 1, lds1);
      compute_tile(lds0);
      wait_all();
      __syncthreads();
      if (kt + 1 < nfull) {
        if (kt + 2 < nfull) issue_tile(kt + 2, lds0);
        compute_tile(lds1);
        wait_all();
        __syncthreads();
      }
    }
  }
  // K tail (K % 64 != 0): one more tile, zero-filled past K, outside the pipelined loop.
  if (nfull * 64 < p.K) {
    guarded_tile(nfull, lds0);
    wait_all();
    __syncthreads();
    compute_tile(lds0);
  }

  // epilogue: lane owns row m = .. + l32 and, per register group rg, columns n .. n+3
  float alpha = 1.f;
  if (p.a_scale) alpha *= *p.a_scale;
  if (p.b_scale) alpha *= *p.b_scale;
  const bool leaky = p.activation == 1;
  const bool vec_ok = p.c_vec_ok;
#pragma unroll
  for (int i = 0; i < MT; i++) {
    int m = m0 + wm * TM + i * 32 + l32;
    if (m >= p.M) continue;
#pragma unroll
    for (int j = 0; j < NT; j++) {
#pragma unroll
      for (int rg = 0; rg < 4; rg++) {
        int n = n0 + wn * TN + j * 32 + rg * 8 + g * 4;
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
          float x = acc[i][j][rg * 4 + e] * alpha;
          if (leaky) x = x >= 0.f ? x : 0.01f * x;
          v[e] = x;
        }
        if (p.out_dtype == 4) {
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
      }
    }
  }
}

template <typename T, int BM, int BN, int WM, int WN, bool B_KMAJOR>
static int launch_one(const GemmArgs& p, hipStream_t stream) {
  constexpr int smem = 2 * (BM + BN) * 128;
  static bool attr_set = false;  // benign race: setting the attribute twice is harmless
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)gemm16_kernel<T, BM, BN, WM, WN, B_KMAJOR>, hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) return (int)e;
    attr_set = true;
  }
  int num_m = (p.M + BM - 1) / BM, num_n = (p.N + BN - 1) / BN;
  gemm16_kernel<T, BM, BN, WM, WN, B_KMAJOR><<<dim3(num_m * num_n), dim3(WM * WN * 64), smem, stream>>>(p);
  return (int)hipGetLastError();
}

template <typename T, bool B_KMAJOR>
static int launch_tile(const GemmArgs& p, int tile, hipStream_t stream) {
  switch (tile) {
    case 0: return launch_one<T, 256, 256, 2, 4, B_KMAJOR>(p, stream);
    case 1: return launch_one<T, 128, 128, 2, 2, B_KMAJOR>(p, stream);
    default: return launch_one<T, 256, 256, 2, 2, B_KMAJOR>(p, stream);
  }
}

// tile: 0 = 256x256 / 8 waves, 1 = 128x128 / 4 waves, 2 = 256x256 / 4 waves
int gemm16_launch(const GemmArgs& p, bool bf16, bool b_kmajor, int tile, hipStream_t stream) {
  if (bf16) return b_kmajor ? launch_tile<__bf16, true>(p, tile, stream) : launch_tile<__bf16, false>(p, tile, stream);
  return b_kmajor ? launch_tile<_Float16, true>(p, tile, stream) : launch_tile<_Float16, false>(p, tile, stream);
}

}  // namespace mi355

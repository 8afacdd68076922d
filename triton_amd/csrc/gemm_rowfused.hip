// One-launch GEMM with the row-wise epilogues of the reference's dot test
// (python/test/unit/language/test_core.py:3128-3145): z = A @ B (+ addend, activation), then optionally
// DO_SOFTMAX (:3136-3141: z - rowmax, exp, divide by the row sum) and / or CHAIN_DOT (:3142-3144:
// `dot(z.to(w.dtype), w)`), and ONE rounding at the store (:3145) - all inside the tile, as the reference
// does it, for products whose row fits one tile: N <= 256 (and, for the chained product, N2 <= 256).
//
// A workgroup of four waves owns 128 rows of C and ALL N columns; each wave 32 rows.  The product is
// computed with the operands swapped (D[n][m], 32x32x16 MFMAs), so a lane holds 16 values of ONE row of z
// per 32-column tile and the pair of lanes (l, l + 32) a whole row: row maximum and row sum are in-lane
// reductions plus one 32-lane swap, and z never leaves the registers.  For the chained product the rounded z
// registers are directly the B operand of out^T = W^T z^T (the K order they imply - rows 4 g .. 4 g + 3 and
// 8 + 4 g .. of each 16 - is applied to the W^T fragments instead), the same register-level hand-over the
// attention kernels use for P.  Operand tiles go through LDS in K chunks of 32 with plain loads (any
// strides, zero-filled edges), fetched into registers one chunk ahead: these are small products, bound by launch
// and latency, not by the MFMA pipe.
#include "common.h"
#include "launch.h"

namespace mi355 {

template <typename V8> struct ElemRF;
template <> struct ElemRF<bf16x8> { using type = __bf16; };
template <> struct ElemRF<f16x8> { using type = _Float16; };

template <typename V8>
__global__ __launch_bounds__(256, 1) void gemm_rowfused_kernel(RowFusedArgs p) {
  using S = typename ElemRF<V8>::type;
  typedef __attribute__((ext_vector_type(4))) S S4;
  constexpr int BM = 128, BK = 32, NTILE = 8, PITCH = BK + 8;   // LDS rows of 40 elements (80 bytes)
  __shared__ __attribute__((aligned(16))) S As[BM][PITCH];
  __shared__ __attribute__((aligned(16))) S Bs[256][PITCH];     // B^T chunk [n][k]; later W^T chunk [n2][n]

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, g = lane >> 5;
  const int m0 = blockIdx.x * BM;
  const S* A = (const S*)p.A;
  const S* B = (const S*)p.B;
  const int ntiles = (p.N + 31) / 32;

  f32x16 acc[NTILE];
#pragma unroll
  for (int j = 0; j < NTILE; j++)
#pragma unroll
    for (int r = 0; r < 16; r++) acc[j][r] = 0.f;

  // ---- z = A @ B over K chunks of 32.  The chunk's operands are fetched into registers one chunk ahead of the MFMAs
  // (all loads of a chunk in flight at once: clamped addresses and a select instead of a branch per element, which
  // the compiler would serialise - one memory round trip per element), then written to LDS.
  // A: (row, group of 8 k) pairs, two per thread.  B, stored transposed in LDS ([n][k]): K-contiguous B as (n, group
  // of 8 k) pairs like A; N-contiguous B as (k, group of 8 n) pairs, 16 bytes along n per load, with k running over the
  // lanes so that the eight 2-byte LDS writes of a lane's values go to consecutive addresses across the wave.
  const bool b_rows = p.sbn == 1 && p.sbk != 1;   // N-contiguous (row-major) B
  V8 ra[2], rb[4];
  auto zero8 = []() { V8 v; for (int e = 0; e < 8; e++) v[e] = (S)0.f; return v; };
  auto gather8 = [&](const S* base, int64_t stride, int first, int limit) {   // elements first .. first + 7 of a line, zeros from `limit` on
    S t[8];
#pragma unroll
    for (int e = 0; e < 8; e++) t[e] = base[(int64_t)min(first + e, limit - 1) * stride];
    V8 v;
#pragma unroll
    for (int e = 0; e < 8; e++) v[e] = first + e < limit ? t[e] : (S)0.f;
    return v;
  };
  auto fetch = [&](int k0) {
#pragma unroll
    for (int i = 0; i < 2; i++) {
      const int idx = tid + i * 256, row = idx >> 2, kg = idx & 3;
      const int m = m0 + row, k = k0 + kg * 8;
      ra[i] = zero8();
      if (m < p.M && k < p.K) {
        const S* src = A + (int64_t)m * p.sam;
        if (p.sak == 1 && k + 8 <= p.K && ((uintptr_t)(src + k) & 15) == 0) ra[i] = *(const V8*)(src + k);
        else ra[i] = gather8(src, p.sak, k, p.K);
      }
    }
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int idx = tid + i * 256;
      rb[i] = zero8();
      if (b_rows) {
        const int kk = idx & 31, n = (idx >> 5) * 8, k = k0 + kk;
        if (k < p.K && n < p.N) {
          const S* src = B + (int64_t)k * p.sbk;
          if (n + 8 <= p.N && ((uintptr_t)(src + n) & 15) == 0) rb[i] = *(const V8*)(src + n);
          else rb[i] = gather8(src, 1, n, p.N);
        }
      } else {
        const int n = idx & 255, k = k0 + (idx >> 8) * 8;
        if (n < p.N && k < p.K) {
          const S* src = B + (int64_t)n * p.sbn;
          if (p.sbk == 1 && k + 8 <= p.K && ((uintptr_t)(src + k) & 15) == 0) rb[i] = *(const V8*)(src + k);
          else rb[i] = gather8(src, p.sbk, k, p.K);
        }
      }
    }
  };
  auto stash = [&]() {
#pragma unroll
    for (int i = 0; i < 2; i++) {
      const int idx = tid + i * 256;
      *(V8*)&As[idx >> 2][(idx & 3) * 8] = ra[i];
    }
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int idx = tid + i * 256;
      if (b_rows) {
        const int kk = idx & 31, n = (idx >> 5) * 8;
#pragma unroll
        for (int e = 0; e < 8; e++) Bs[n + e][kk] = rb[i][e];
      } else {
        *(V8*)&Bs[idx & 255][(idx >> 8) * 8] = rb[i];
      }
    }
  };
  fetch(0);
  for (int k0 = 0; k0 < p.K; k0 += BK) {
    stash();
    __syncthreads();
    if (k0 + BK < p.K) fetch(k0 + BK);
#pragma unroll
    for (int ks = 0; ks < 2; ks++) {
      const V8 af = *(const V8*)&As[wave * 32 + l32][ks * 16 + g * 8];
      static_for<NTILE>([&](auto J_) {
        constexpr int j = decltype(J_)::value;
        if (j < ntiles) {
          const V8 bf = *(const V8*)&Bs[j * 32 + l32][ks * 16 + g * 8];
          acc[j] = mfma32(bf, af, acc[j]);   // D[n][m]: lane l32 <-> row m, registers <-> columns n
        }
      });
    }
    __syncthreads();
  }

  // ---- epilogue on the registers: register r of tile j is column n = 32 j + 8 (r / 4) + 4 g + r % 4 of row m
  const int m = m0 + wave * 32 + l32;
  const bool row_ok = m < p.M;
  float alpha = 1.f;
  if (p.a_scale) alpha *= *p.a_scale;
  if (p.b_scale) alpha *= *p.b_scale;
  auto col = [&](int j, int r) { return 32 * j + 8 * (r >> 2) + 4 * g + (r & 3); };
  // (everything below touches the tiles j < ntiles only, and the addend / activation / softmax code only when asked
  // for: these are small products whose time is the code they execute - and fetch: the reference's timing protocol
  // flushes the caches, instructions included, before every call)
  const bool has_aux = p.aux != nullptr, leaky = p.activation == 1;
  static_for<NTILE>([&](auto J_) {
    constexpr int j = decltype(J_)::value;
    if (j < ntiles) {
#pragma unroll
      for (int r = 0; r < 16; r++) acc[j][r] *= alpha;
      if (has_aux) {
#pragma unroll
        for (int r = 0; r < 16; r++) {
          const int n = col(j, r);
          if (row_ok && n < p.N) acc[j][r] += load_aux(p.aux, (int64_t)m * p.aux_sm + (int64_t)n * p.aux_sn, p.aux_dtype);
        }
      }
      if (leaky) {
#pragma unroll
        for (int r = 0; r < 16; r++) acc[j][r] = acc[j][r] >= 0.f ? acc[j][r] : 0.01f * acc[j][r];
      }
    }
  });
  if (p.softmax) {
    float mx = -INFINITY;
    static_for<NTILE>([&](auto J_) {
      constexpr int j = decltype(J_)::value;
      if (j < ntiles) {
#pragma unroll
        for (int r = 0; r < 16; r++) if (col(j, r) < p.N) mx = fmaxf(mx, acc[j][r]);
      }
    });
    mx = pair_max(mx);
    float sum = 0.f;
    static_for<NTILE>([&](auto J_) {
      constexpr int j = decltype(J_)::value;
      if (j < ntiles) {
#pragma unroll
        for (int r = 0; r < 16; r++) {
          const float e = col(j, r) < p.N ? __expf(acc[j][r] - mx) : 0.f;
          acc[j][r] = e;
          sum += e;
        }
      }
    });
    sum = pair_sum(sum);
    const float inv = 1.f / sum;
    static_for<NTILE>([&](auto J_) {
      constexpr int j = decltype(J_)::value;
      if (j < ntiles) {
#pragma unroll
        for (int r = 0; r < 16; r++) acc[j][r] *= inv;
      }
    });
  }

  auto store_row4 = [&](const float (&v)[4], int n, int ncols) {   // four consecutive columns n .. n + 3 of row m
    if (!row_ok) return;
    const int64_t off0 = (int64_t)m * p.scm + (int64_t)n * p.scn;
    if (p.scn == 1 && n + 4 <= ncols) {   // one store of four values where the row lets it
      if (p.out_dtype == 4) {
        float* c = (float*)p.C + off0;
        if (((uintptr_t)c & 15) == 0) { *(f32x4*)c = f32x4{v[0], v[1], v[2], v[3]}; return; }
      } else if (p.out_dtype == 1) {
        __bf16* c = (__bf16*)p.C + off0;
        if (((uintptr_t)c & 7) == 0) { *(bf16x4*)c = bf16x4{(__bf16)v[0], (__bf16)v[1], (__bf16)v[2], (__bf16)v[3]}; return; }
      } else {
        _Float16* c = (_Float16*)p.C + off0;
        if (((uintptr_t)c & 7) == 0) { *(f16x4*)c = f16x4{(_Float16)v[0], (_Float16)v[1], (_Float16)v[2], (_Float16)v[3]}; return; }
      }
    }
#pragma unroll
    for (int e = 0; e < 4; e++) {
      if (n + e >= ncols) continue;
      const int64_t off = off0 + (int64_t)e * p.scn;
      if (p.out_dtype == 4) ((float*)p.C)[off] = v[e];
      else if (p.out_dtype == 1) ((__bf16*)p.C)[off] = (__bf16)v[e];
      else ((_Float16*)p.C)[off] = (_Float16)v[e];
    }
  };

  if (!p.W) {
    static_for<NTILE>([&](auto J_) {
      constexpr int j = decltype(J_)::value;
      if (j < ntiles) {
#pragma unroll
        for (int rg = 0; rg < 4; rg++) {
          const float v[4] = {acc[j][rg * 4], acc[j][rg * 4 + 1], acc[j][rg * 4 + 2], acc[j][rg * 4 + 3]};
          store_row4(v, 32 * j + 8 * rg + 4 * g, p.N);
        }
      }
    });
    return;
  }

  // ---- chained product: out[m][n2] = sum_n z^[m][n] W[n][n2], z^ = z rounded to the operand type.
  // zf[j][t] = registers 8 t .. 8 t + 7 of tile j as a B operand: K slots e < 4 are n = 32 j + 16 t + 4 g + e,
  // slots e >= 4 are n = 32 j + 16 t + 8 + 4 g + (e - 4)
  V8 zf[NTILE][2];
  static_for<NTILE>([&](auto J_) {
    constexpr int j = decltype(J_)::value;
    if (j < ntiles) {
#pragma unroll
      for (int t = 0; t < 2; t++)
#pragma unroll
        for (int e = 0; e < 8; e++) zf[j][t][e] = (S)(col(j, t * 8 + e) < p.N ? acc[j][t * 8 + e] : 0.f);
    }
  });
  const S* W = (const S*)p.W;
  const int n2tiles = (p.N2 + 31) / 32;
  f32x16 out[NTILE];
#pragma unroll
  for (int j = 0; j < NTILE; j++)
#pragma unroll
    for (int r = 0; r < 16; r++) out[j][r] = 0.f;
  static_for<NTILE>([&](auto J_) {
    constexpr int j = decltype(J_)::value;   // chunk of 32 rows n of W
    if (j < ntiles) {
      __syncthreads();
      // W^T chunk [n2][n local]: (n2, group of 8 n) pairs, four per thread
#pragma unroll
      for (int i = 0; i < 4; i++) {
        const int idx = tid + i * 256, n2 = idx & 255, ng = idx >> 8;
        // (all eight loads in flight at once: clamped addresses, then a select)
        S t[8];
#pragma unroll
        for (int e = 0; e < 8; e++) t[e] = W[(int64_t)min(32 * j + ng * 8 + e, p.N - 1) * p.swn + (int64_t)min(n2, p.N2 - 1) * p.swn2];
        V8 v;
#pragma unroll
        for (int e = 0; e < 8; e++) v[e] = (n2 < p.N2 && 32 * j + ng * 8 + e < p.N) ? t[e] : (S)0.f;
        *(V8*)&Bs[n2][ng * 8] = v;
      }
      __syncthreads();
#pragma unroll
      for (int t = 0; t < 2; t++) {
        static_for<NTILE>([&](auto J2_) {
          constexpr int j2 = decltype(J2_)::value;
          if (j2 < n2tiles) {
            const S4 lo = *(const S4*)&Bs[j2 * 32 + l32][16 * t + 4 * g];
            const S4 hi = *(const S4*)&Bs[j2 * 32 + l32][16 * t + 8 + 4 * g];
            const V8 wf = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            out[j2] = mfma32(wf, zf[j][t], out[j2]);   // D[n2][m]
          }
        });
      }
    }
  });
  static_for<NTILE>([&](auto J_) {
    constexpr int j = decltype(J_)::value;
    if (j < n2tiles) {
#pragma unroll
      for (int rg = 0; rg < 4; rg++) {
        const float v[4] = {out[j][rg * 4], out[j][rg * 4 + 1], out[j][rg * 4 + 2], out[j][rg * 4 + 3]};
        store_row4(v, 32 * j + 8 * rg + 4 * g, p.N2);
      }
    }
  });
}

int gemm_rowfused_launch(const RowFusedArgs& p, bool bf16, hipStream_t stream) {
  const dim3 grid((p.M + 127) / 128), block(256);
  if (bf16) gemm_rowfused_kernel<bf16x8><<<grid, block, 0, stream>>>(p);
  else gemm_rowfused_kernel<f16x8><<<grid, block, 0, stream>>>(p);
  return (int)hipGetLastError();
}

}  // namespace mi355

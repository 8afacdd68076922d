// Flash-attention backward for gfx950 (fp16 / bf16, head_dim 64 or 128): delta = rowsum(O*dO),
// then dK/dV with the K/V tile stationary and dQ with the Q tile stationary - the same
// atomics-free split as the reference (`_attn_bwd_preprocess`, `_attn_bwd_dkdv`, `_attn_bwd_dq`,
// python/tutorials/06-fused-attention.py:190-204, :208-257, :261-305, driver :308-435), as
// separate launches.
//
// Per (query row m, key row n), with s2 = sm_scale * log2(e) and M the forward's base-2
// log-sum-exp:   p = exp2(q.k * s2 - M[m])        (:235-236 / :288)
//                dv[n] += p^ * do[m]               (p^ = p rounded to the input type, :243-245)
//                dp = do[m].v[n];  ds = p * (dp - delta[m])   (:247-250 / :294-296)
//                dk[n] += ds^ * q[m] * sm_scale;   dq[m] += ds^ * k[n] * sm_scale
// The reference folds s2 into K on the host, rounded to the input type (:490-492), and undoes
// it with ln2 / sm_scale factors (:386, :434); here K stays as given and the factors are
// applied in fp32.  causal = 0 runs the full rectangle, which the reference kernel cannot
// (its backward always applies the causal bounds).
//
// Operand plan (32x32x16 MFMA, lane l <-> column l%32, accumulator registers <-> rows):
//   dQ kernel:    S^T = K Q^T and dP^T = V dO^T put one query row per lane, so M and delta are
//                 per-lane scalars and ds^T is directly the B operand of dQ^T = K^T ds^T;
//                 Q and dO fragments stay in registers, K / V tiles stream through LDS.
//   dK/dV kernel: S = Q K^T and dP = dO V^T put one key row per lane, p and ds are directly
//                 the B operands of dV^T = dO^T p and dK^T = Q^T ds; K and V fragments stay in
//                 registers, Q / dO tiles stream through LDS.
// Every streamed tile is read both row-wise (ds_read_b128) and transposed
// (ds_read_b64_tr_b16); one XOR swizzle (attn_tiles.h) serves both access patterns.
#include "attn_tiles.h"
#include "launch.h"

namespace mi355 {

template <typename V8> struct ElemB;
template <> struct ElemB<bf16x8> { using type = __bf16; };
template <> struct ElemB<f16x8> { using type = _Float16; };

// ---------------------------------------------------------------------------------------------
// delta[hz, m] = sum_d o[m,d] * do[m,d]   (fp32)
// ---------------------------------------------------------------------------------------------
template <typename V8, int D>
__global__ __launch_bounds__(256) void attn_bwd_pre_kernel(AttnArgs p) {
  constexpr int LPR = D / 8;  // lanes per row, 16 bytes each
  const int rows_per_block = 256 / LPR;
  const int row = blockIdx.x * rows_per_block + threadIdx.x / LPR;
  const int hz = blockIdx.y, z = hz / p.H, h = hz % p.H;
  const int c = threadIdx.x % LPR;
  float acc = 0.f;
  if (row < p.N) {
    int64_t off = ((int64_t)z * p.so[0] + (int64_t)h * p.so[1] + (int64_t)row * p.so[2]) * 2 + c * 16;
    V8 o = *(const V8*)(p.o + off);
    V8 d = *(const V8*)(p.d_o + off);
#pragma unroll
    for (int e = 0; e < 8; e++) acc = fmaf((float)o[e], (float)d[e], acc);
  }
#pragma unroll
  for (int s = LPR / 2; s >= 1; s >>= 1) acc += __shfl_xor(acc, s);
  if (row < p.N && c == 0) p.lse[(int64_t)hz * p.N + row] = acc;
}

// ---------------------------------------------------------------------------------------------
// dQ: one wave owns QT*32 query rows; K / V tiles of 64 rows stream through LDS.
// ---------------------------------------------------------------------------------------------
template <typename V8, int D, int QT, int NW>
__global__ __launch_bounds__(NW * 64, 1) void attn_bwd_dq_kernel(AttnArgs p) {
  using S = typename ElemB<V8>::type;
  typedef __attribute__((ext_vector_type(4))) S S4;
  constexpr int BM = NW * QT * 32, BN = 64, RB = D * 2, KSQ = D / 16, DT = D / 32;
  using Tile = AttnTile<RB, BN, NW>;
  constexpr int TILE = Tile::BYTES;

  extern __shared__ __attribute__((aligned(1024))) char smem[];
  LDS_PTR(char) const lds = (LDS_PTR(char))smem;  // [stage][K tile | V tile]

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, g = lane >> 5, i16 = lane & 15, q4 = lane >> 4;

  const int nqb = (p.N + BM - 1) / BM;
  int pid = xcd_remap(blockIdx.x, nqb * p.Z * p.H);
  const int hz = pid / nqb;
  int qb = pid % nqb;
  if (p.causal) qb = nqb - 1 - qb;
  const int z = hz / p.H, h = hz % p.H;
  const int m0 = qb * BM, row0 = m0 + wave * QT * 32;

  const int64_t head_off = ((int64_t)z * p.sq[0] + (int64_t)h * p.sq[1]) * 2;
  const int64_t pitch = p.sq[2] * 2;
  const char* qbase = p.q + head_off;
  const char* kbase = p.k + head_off;
  const char* vbase = p.v + head_off;
  const char* dobase = p.d_o + head_off;

  V8 qf[QT][KSQ], dof[QT][KSQ];
  float m_row[QT], d_row[QT];
#pragma unroll
  for (int b = 0; b < QT; b++) {
    int r = min(row0 + b * 32 + l32, p.N - 1);
    const char* sq = qbase + (int64_t)r * pitch + g * 16;
    const char* sd = dobase + (int64_t)r * pitch + g * 16;
#pragma unroll
    for (int ks = 0; ks < KSQ; ks++) {
      qf[b][ks] = *(const V8*)(sq + ks * 32);
      dof[b][ks] = *(const V8*)(sd + ks * 32);
    }
    m_row[b] = p.lse[(int64_t)hz * p.N + r];
    d_row[b] = p.delta[(int64_t)hz * p.N + r];
  }

  const char* srcK[Tile::INST];
  const char* srcV[Tile::INST];
#pragma unroll
  for (int i = 0; i < Tile::INST; i++) {
    srcK[i] = Tile::src(kbase, pitch, wave, lane, i);
    srcV[i] = Tile::src(vbase, pitch, wave, lane, i);
  }
  auto issue_kv = [&](int j, int stage) {
    LDS_PTR(char) kd = lds + stage * (2 * TILE);
    LDS_PTR(char) vd = kd + TILE;
#pragma unroll
    for (int i = 0; i < Tile::INST; i++) {
      async_copy16(srcK[i] + (int64_t)j * BN * pitch, (LDS_PTR(void))(kd + (i * NW + wave) * 1024));
      async_copy16(srcV[i] + (int64_t)j * BN * pitch, (LDS_PTR(void))(vd + (i * NW + wave) * 1024));
    }
  };

  const RowRead<RB> rr(l32, g);
  const TrRead<RB> tt(i16, q4);

  f32x16 dq[DT][QT];
#pragma unroll
  for (int c = 0; c < DT; c++)
#pragma unroll
    for (int b = 0; b < QT; b++)
#pragma unroll
      for (int r = 0; r < 16; r++) dq[c][b][r] = 0.f;

  const float qk_scale = p.sm_scale * 1.4426950408889634f;
  const int kv_end_blk = p.causal ? min(p.N, m0 + BM) : p.N;
  const int nsteps = (kv_end_blk + BN - 1) / BN;
  const int wave_last = p.causal ? (row0 + QT * 32 - 1) / BN : nsteps - 1;
  const int wave_first_masked = p.causal ? row0 / BN : nsteps;

  issue_kv(0, 0);
  wait_all();
  __syncthreads();

  for (int j = 0; j < nsteps; j++) {
    const int stage = j & 1;
    if (j + 1 < nsteps) issue_kv(j + 1, stage ^ 1);
    if (j <= wave_last && row0 < p.N) {
      const unsigned kb = lds_addr(lds + stage * (2 * TILE));
      const unsigned vb = kb + TILE;
      V8 dsf[QT][4];
#pragma unroll
      for (int a = 0; a < 2; a++) {
        // S^T and dP^T for key tile a: [QT q tiles]
        f32x16 s[QT], dp[QT];
#pragma unroll
        for (int b = 0; b < QT; b++)
#pragma unroll
          for (int r = 0; r < 16; r++) { s[b][r] = 0.f; dp[b][r] = 0.f; }
        i32x4 kf[2], vf[2];
        kf[0] = a == 0 ? lds_read_b128<0>(rr.template addr<0>(kb)) : lds_read_b128<32 * RB>(rr.template addr<0>(kb));
        vf[0] = a == 0 ? lds_read_b128<0>(rr.template addr<0>(vb)) : lds_read_b128<32 * RB>(rr.template addr<0>(vb));
        static_for<KSQ>([&](auto KS_) {
          constexpr int ks = decltype(KS_)::value;
          constexpr int cur = ks & 1, nxt = cur ^ 1;
          if constexpr (ks + 1 < KSQ) {
            kf[nxt] = a == 0 ? lds_read_b128<0>(rr.template addr<ks + 1>(kb)) : lds_read_b128<32 * RB>(rr.template addr<ks + 1>(kb));
            vf[nxt] = a == 0 ? lds_read_b128<0>(rr.template addr<ks + 1>(vb)) : lds_read_b128<32 * RB>(rr.template addr<ks + 1>(vb));
            lds_wait<2>();
          } else {
            lds_wait<0>();
          }
          lds_use(kf[cur]);
          lds_use(vf[cur]);
#pragma unroll
          for (int b = 0; b < QT; b++) {
            s[b] = mfma32(__builtin_bit_cast(V8, kf[cur]), qf[b][ks], s[b]);
            dp[b] = mfma32(__builtin_bit_cast(V8, vf[cur]), dof[b][ks], dp[b]);
          }
        });
#pragma unroll
        for (int b = 0; b < QT; b++) {
          const int qrow = row0 + b * 32 + l32;
          const bool masked = j >= wave_first_masked;
#pragma unroll
          for (int r = 0; r < 16; r++) {
            float pv = fast_exp2(fmaf(s[b][r], qk_scale, -m_row[b]));
            if (masked) {
              int kv = j * BN + a * 32 + (r >> 2) * 8 + g * 4 + (r & 3);
              if (kv > qrow) pv = 0.f;
            }
            float dsv = pv * (dp[b][r] - d_row[b]);
            dsf[b][a * 2 + (r >> 3)][r & 7] = (S)dsv;
          }
        }
      }
      // dQ^T += K^T ds^T : [DT d tiles][QT q tiles], 4 k-steps of 16 key rows
      {
        i32x2 tf[2][DT][2];
        auto read_t = [&](auto T_, i32x2 (&dst)[DT][2]) {
          constexpr int t = decltype(T_)::value;
          static_for<DT>([&](auto C_) {
            constexpr int c = decltype(C_)::value;
            dst[c][0] = lds_read_tr16_b64<16 * t * RB>(tt.template addr<c, 0>(kb));
            dst[c][1] = lds_read_tr16_b64<(16 * t + 8) * RB>(tt.template addr<c, 1>(kb));
          });
        };
        read_t(std::integral_constant<int, 0>{}, tf[0]);
        static_for<4>([&](auto T_) {
          constexpr int t = decltype(T_)::value;
          constexpr int cur = t & 1, nxt = cur ^ 1;
          if constexpr (t + 1 < 4) {
            read_t(std::integral_constant<int, t + 1>{}, tf[nxt]);
            lds_wait<2 * DT>();
          } else {
            lds_wait<0>();
          }
#pragma unroll
          for (int c = 0; c < DT; c++) {
            lds_use(tf[cur][c][0]);
            lds_use(tf[cur][c][1]);
            i32x4 both = __builtin_shufflevector(tf[cur][c][0], tf[cur][c][1], 0, 1, 2, 3);
#pragma unroll
            for (int b = 0; b < QT; b++) dq[c][b] = mfma32(__builtin_bit_cast(V8, both), dsf[b][t], dq[c][b]);
          }
        });
      }
    }
    wait_all();
    __syncthreads();
  }

#pragma unroll
  for (int b = 0; b < QT; b++) {
    const int row = row0 + b * 32 + l32;
    if (row >= p.N) continue;
    char* dst = p.dq + head_off + (int64_t)row * pitch;
#pragma unroll
    for (int c = 0; c < DT; c++)
#pragma unroll
      for (int rg = 0; rg < 4; rg++) {
        int d = c * 32 + rg * 8 + g * 4;
        S4 v;
#pragma unroll
        for (int e = 0; e < 4; e++) v[e] = (S)(dq[c][b][rg * 4 + e] * p.sm_scale);
        *(S4*)(dst + d * 2) = v;
      }
  }
}

// ---------------------------------------------------------------------------------------------
// dK/dV: one wave owns 32 key rows; Q / dO tiles of 64 rows stream through LDS.
// ---------------------------------------------------------------------------------------------
template <typename V8, int D, int NW>
__global__ __launch_bounds__(NW * 64, 1) void attn_bwd_dkdv_kernel(AttnArgs p) {
  using S = typename ElemB<V8>::type;
  typedef __attribute__((ext_vector_type(4))) S S4;
  constexpr int BN = NW * 32, BM = 64, MT = BM / 32, RB = D * 2, KSQ = D / 16, DT = D / 32;
  using Tile = AttnTile<RB, BM, NW>;
  constexpr int TILE = Tile::BYTES;

  extern __shared__ __attribute__((aligned(1024))) char smem[];
  LDS_PTR(char) const lds = (LDS_PTR(char))smem;  // [stage][Q tile | dO tile | M rows | delta rows]
  constexpr int STAGE = 2 * Tile::BYTES + 2 * BM * 4;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
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
      kf[ks] = *(const V8*)(sk + ks * 32);
      vf[ks] = *(const V8*)(sv + ks * 32);
    }
  }

  const char* srcQ[Tile::INST];
  const char* srcD[Tile::INST];
#pragma unroll
  for (int i = 0; i < Tile::INST; i++) {
    srcQ[i] = Tile::src(qbase, pitch, wave, lane, i);
    srcD[i] = Tile::src(dobase, pitch, wave, lane, i);
  }
  // the M and delta values of the tile's query rows ride along (4 bytes per lane: wave 0 copies
  // the 64 M values, wave 1 the 64 deltas), so the loop issues no register loads that would have to
  // wait behind the tile copies
  const float* src_stat = (wave == 0 ? lse : delta) + lane;
  auto issue_qd = [&](int mstart, int stage) {
    LDS_PTR(char) qd = lds + stage * STAGE;
    LDS_PTR(char) dd = qd + TILE;
#pragma unroll
    for (int i = 0; i < Tile::INST; i++) {
      async_copy16(srcQ[i] + (int64_t)mstart * pitch, (LDS_PTR(void))(qd + (i * NW + wave) * 1024));
      async_copy16(srcD[i] + (int64_t)mstart * pitch, (LDS_PTR(void))(dd + (i * NW + wave) * 1024));
    }
    if (wave < 2) async_copy4(src_stat + mstart, (LDS_PTR(void))(qd + 2 * TILE + wave * (BM * 4)));
  };

  const RowRead<RB> rr(l32, g);
  const TrRead<RB> tt(i16, q4);

  f32x16 dk[DT], dv[DT];
#pragma unroll
  for (int c = 0; c < DT; c++)
#pragma unroll
    for (int r = 0; r < 16; r++) { dk[c][r] = 0.f; dv[c][r] = 0.f; }

  const float qk_scale = p.sm_scale * 1.4426950408889634f;
  // query rows m >= n0 (causal) or all of them, in steps of BM
  const int m_begin = p.causal ? (n0 / BM) * BM : 0;
  const int nsteps = (p.N - m_begin + BM - 1) / BM;
  const int ncol = nrow0 + l32;  // this lane's key row

  issue_qd(m_begin, 0);
  wait_all();
  __syncthreads();

  for (int j = 0; j < nsteps; j++) {
    const int stage = j & 1;
    const int ms = m_begin + j * BM;
    if (j + 1 < nsteps) issue_qd(ms + BM, stage ^ 1);
    if (nrow0 < p.N) {
      const unsigned qb = lds_addr(lds + stage * STAGE);
      const unsigned db = qb + TILE;
      const unsigned sb = qb + 2 * TILE + g * 16;
#pragma unroll
      for (int mt = 0; mt < MT; mt++) {
        const int mrow0 = ms + mt * 32;
        // causal: rows below this wave's first key row contribute nothing
        if (p.causal && mrow0 + 31 < nrow0) continue;
        const bool masked = p.causal && mrow0 < nrow0 + 31;
        // M and delta of the 16 query rows this lane's registers stand for
        i32x4 mvi[4], dli[4];
        static_for<4>([&](auto RG_) {
          constexpr int rg = decltype(RG_)::value;
          if (mt == 0) {
            mvi[rg] = lds_read_b128<rg * 32>(sb);
            dli[rg] = lds_read_b128<BM * 4 + rg * 32>(sb);
          } else {
            mvi[rg] = lds_read_b128<128 + rg * 32>(sb);
            dli[rg] = lds_read_b128<BM * 4 + 128 + rg * 32>(sb);
          }
        });
        f32x16 s, dp;
#pragma unroll
        for (int r = 0; r < 16; r++) { s[r] = 0.f; dp[r] = 0.f; }
        {
          i32x4 qf[2], df[2];
          qf[0] = mt == 0 ? lds_read_b128<0>(rr.template addr<0>(qb)) : lds_read_b128<32 * RB>(rr.template addr<0>(qb));
          df[0] = mt == 0 ? lds_read_b128<0>(rr.template addr<0>(db)) : lds_read_b128<32 * RB>(rr.template addr<0>(db));
          static_for<KSQ>([&](auto KS_) {
            constexpr int ks = decltype(KS_)::value;
            constexpr int cur = ks & 1, nxt = cur ^ 1;
            if constexpr (ks + 1 < KSQ) {
              qf[nxt] = mt == 0 ? lds_read_b128<0>(rr.template addr<ks + 1>(qb)) : lds_read_b128<32 * RB>(rr.template addr<ks + 1>(qb));
              df[nxt] = mt == 0 ? lds_read_b128<0>(rr.template addr<ks + 1>(db)) : lds_read_b128<32 * RB>(rr.template addr<ks + 1>(db));
              lds_wait<2>();
            } else {
              lds_wait<0>();
            }
            lds_use(qf[cur]);
            lds_use(df[cur]);
            if constexpr (ks + 1 == KSQ) {
#pragma unroll
              for (int rg = 0; rg < 4; rg++) { lds_use(mvi[rg]); lds_use(dli[rg]); }
            }
            s = mfma32(__builtin_bit_cast(V8, qf[cur]), kf[ks], s);    // S[m][n]
            dp = mfma32(__builtin_bit_cast(V8, df[cur]), vf[ks], dp);  // dP[m][n]
          });
        }
        f32x4 mv[4], dl[4];
#pragma unroll
        for (int rg = 0; rg < 4; rg++) {
          mv[rg] = __builtin_bit_cast(f32x4, mvi[rg]);
          dl[rg] = __builtin_bit_cast(f32x4, dli[rg]);
        }
        V8 pf[2], dsf[2];
#pragma unroll
        for (int r = 0; r < 16; r++) {
          float pv = fast_exp2(fmaf(s[r], qk_scale, -mv[r >> 2][r & 3]));
          if (masked) {
            int m = mrow0 + (r >> 2) * 8 + g * 4 + (r & 3);
            if (m < ncol) pv = 0.f;
          }
          float dsv = pv * (dp[r] - dl[r >> 2][r & 3]);
          pf[r >> 3][r & 7] = (S)pv;
          dsf[r >> 3][r & 7] = (S)dsv;
        }
        // dV^T += dO^T p ; dK^T += Q^T ds : [DT d tiles], 2 k-steps of 16 query rows
        {
          i32x2 tq[2][DT][2], td[2][DT][2];
          auto read_t = [&](auto T_, i32x2 (&dq_)[DT][2], i32x2 (&dd_)[DT][2]) {
            constexpr int t = decltype(T_)::value;
            static_for<DT>([&](auto C_) {
              constexpr int c = decltype(C_)::value;
              constexpr int imm0 = 16 * t * RB;
              if (mt == 0) {
                dq_[c][0] = lds_read_tr16_b64<imm0>(tt.template addr<c, 0>(qb));
                dq_[c][1] = lds_read_tr16_b64<imm0 + 8 * RB>(tt.template addr<c, 1>(qb));
                dd_[c][0] = lds_read_tr16_b64<imm0>(tt.template addr<c, 0>(db));
                dd_[c][1] = lds_read_tr16_b64<imm0 + 8 * RB>(tt.template addr<c, 1>(db));
              } else {
                dq_[c][0] = lds_read_tr16_b64<imm0 + 32 * RB>(tt.template addr<c, 0>(qb));
                dq_[c][1] = lds_read_tr16_b64<imm0 + 40 * RB>(tt.template addr<c, 1>(qb));
                dd_[c][0] = lds_read_tr16_b64<imm0 + 32 * RB>(tt.template addr<c, 0>(db));
                dd_[c][1] = lds_read_tr16_b64<imm0 + 40 * RB>(tt.template addr<c, 1>(db));
              }
            });
          };
          read_t(std::integral_constant<int, 0>{}, tq[0], td[0]);
          static_for<2>([&](auto T_) {
            constexpr int t = decltype(T_)::value;
            constexpr int cur = t & 1, nxt = cur ^ 1;
            if constexpr (t + 1 < 2) {
              read_t(std::integral_constant<int, t + 1>{}, tq[nxt], td[nxt]);
              lds_wait<4 * DT>();
            } else {
              lds_wait<0>();
            }
#pragma unroll
            for (int c = 0; c < DT; c++) {
              lds_use(tq[cur][c][0]); lds_use(tq[cur][c][1]);
              lds_use(td[cur][c][0]); lds_use(td[cur][c][1]);
              i32x4 qt = __builtin_shufflevector(tq[cur][c][0], tq[cur][c][1], 0, 1, 2, 3);
              i32x4 dt = __builtin_shufflevector(td[cur][c][0], td[cur][c][1], 0, 1, 2, 3);
              dv[c] = mfma32(__builtin_bit_cast(V8, dt), pf[t], dv[c]);
              dk[c] = mfma32(__builtin_bit_cast(V8, qt), dsf[t], dk[c]);
            }
          });
        }
      }
    }
    wait_all();
    __syncthreads();
  }

  if (ncol < p.N) {
    char* dkd = p.dk + head_off + (int64_t)ncol * pitch;
    char* dvd = p.dv + head_off + (int64_t)ncol * pitch;
#pragma unroll
    for (int c = 0; c < DT; c++)
#pragma unroll
      for (int rg = 0; rg < 4; rg++) {
        int d = c * 32 + rg * 8 + g * 4;
        S4 a, b;
#pragma unroll
        for (int e = 0; e < 4; e++) {
          a[e] = (S)(dk[c][rg * 4 + e] * p.sm_scale);
          b[e] = (S)dv[c][rg * 4 + e];
        }
        *(S4*)(dkd + d * 2) = a;
        *(S4*)(dvd + d * 2) = b;
      }
  }
}

template <typename V8, int D>
static int launch_bwd_d(const AttnArgs& p, hipStream_t stream) {
  {
    constexpr int QT = 1, NW = 4, BM = NW * QT * 32;
    constexpr int smem = 2 * 2 * 64 * D * 2;
    static bool attr_set = false;
    if (!attr_set) {
      hipError_t e = hipFuncSetAttribute((const void*)attn_bwd_dq_kernel<V8, D, QT, NW>,
                                         hipFuncAttributeMaxDynamicSharedMemorySize, smem);
      if (e != hipSuccess) return (int)e;
      attr_set = true;
    }
    int nqb = (p.N + BM - 1) / BM;
    attn_bwd_dq_kernel<V8, D, QT, NW><<<dim3(nqb * p.Z * p.H), dim3(NW * 64), smem, stream>>>(p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return (int)e;
  }
  {
    constexpr int NW = 4, BN = NW * 32;
    constexpr int smem = 2 * (2 * 64 * D * 2 + 2 * 64 * 4);
    static bool attr_set = false;
    if (!attr_set) {
      hipError_t e = hipFuncSetAttribute((const void*)attn_bwd_dkdv_kernel<V8, D, NW>,
                                         hipFuncAttributeMaxDynamicSharedMemorySize, smem);
      if (e != hipSuccess) return (int)e;
      attr_set = true;
    }
    int nkb = (p.N + BN - 1) / BN;
    attn_bwd_dkdv_kernel<V8, D, NW><<<dim3(nkb * p.Z * p.H), dim3(NW * 64), smem, stream>>>(p);
    return (int)hipGetLastError();
  }
}

int attn_bwd_launch(const AttnArgs& p, bool bf16, hipStream_t stream) {
  if (bf16) return p.D == 128 ? launch_bwd_d<bf16x8, 128>(p, stream) : launch_bwd_d<bf16x8, 64>(p, stream);
  return p.D == 128 ? launch_bwd_d<f16x8, 128>(p, stream) : launch_bwd_d<f16x8, 64>(p, stream);
}

int attn_bwd_pre_launch(const AttnArgs& p, bool bf16, hipStream_t stream) {
  dim3 grid, block(256);
  if (p.D == 128) {
    grid = dim3((p.N + 15) / 16, p.Z * p.H);
    if (bf16) attn_bwd_pre_kernel<bf16x8, 128><<<grid, block, 0, stream>>>(p);
    else attn_bwd_pre_kernel<f16x8, 128><<<grid, block, 0, stream>>>(p);
  } else {
    grid = dim3((p.N + 31) / 32, p.Z * p.H);
    if (bf16) attn_bwd_pre_kernel<bf16x8, 64><<<grid, block, 0, stream>>>(p);
    else attn_bwd_pre_kernel<f16x8, 64><<<grid, block, 0, stream>>>(p);
  }
  return (int)hipGetLastError();
}

}  // namespace mi355

// Flash-attention backward for gfx950 (fp16 / bf16, head_dim 64, 128 or 256): delta = rowsum(O*dO),
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
  if (row < p.N && c * 8 < p.d_real) {   // (head dims 16 / 32 run the 64-column form: the columns beyond d_real do not exist)
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
// PAD (D = 64 only): p.d_real = 16 or 32 columns exist in memory; fragments loaded into registers are zero-filled,
// the LDS tiles are zeroed once and only the chunks present are loaded, only the first d_real columns are stored.
template <typename V8, int D, int QT, int NW, bool PAD = false>
__global__ __launch_bounds__(NW * 64, 1) void attn_bwd_dq_kernel(AttnArgs p) {
  using S = typename ElemB<V8>::type;
  typedef __attribute__((ext_vector_type(4))) S S4;
  constexpr int BM = NW * QT * 32, BN = 64, RB = D * 2, KSQ = D / 16, DT = D / 32;
  using Tile = AttnTile<RB, BN, NW>;
  constexpr int TILE = Tile::BYTES;

  extern __shared__ __attribute__((aligned(1024))) char smem[];
  LDS_PTR(char) const lds = (LDS_PTR(char))smem;  // [stage][K tile | V tile]

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
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
      if (!PAD || ks * 32 + g * 16 < p.d_real * 2) {
        qf[b][ks] = *(const V8*)(sq + ks * 32);
        dof[b][ks] = *(const V8*)(sd + ks * 32);
      } else {
        qf[b][ks] = V8{};
        dof[b][ks] = V8{};
      }
    }
    m_row[b] = p.lse[(int64_t)hz * p.N + r];
    d_row[b] = p.delta[(int64_t)hz * p.N + r];
  }

  // direct loads: scalar tile base + 32-bit lane offset (the host bounds the row pitch)
  unsigned offKV[Tile::INST];
  bool present[Tile::INST];
#pragma unroll
  for (int i = 0; i < Tile::INST; i++) {
    offKV[i] = (unsigned)Tile::off(pitch, wave, lane, i);
    present[i] = !PAD || Tile::chunk_present(wave, lane, i, p.d_real * 2);
  }
  const unsigned lds_base = lds_addr(lds);
  if constexpr (PAD) {
    lds_zero(lds, 2 * 2 * TILE, tid, NW * 64);
    __syncthreads();
  }
  // the K and V tiles of step j into LDS stage `stage`: 2 * INST loads per wave, as a burst (prologue, waves without
  // work in a step) or one at a time between the MFMAs of the step before
  struct KvSrc { const char* k; const char* v; unsigned lds; };
  auto kv_src = [&](int j, int stage) {
    const int64_t off = (int64_t)j * BN * pitch;
    return KvSrc{kbase + off, vbase + off, lds_base + stage * (2 * TILE)};
  };
  auto kv_load = [&](auto I_, const KvSrc& src) {
    constexpr int I = decltype(I_)::value, i = I >> 1;
    if (present[i]) {
      if constexpr ((I & 1) == 0) async_copy16_sbase(src.k, offKV[i], src.lds + (i * NW + wave) * 1024);
      else async_copy16_sbase(src.v, offKV[i], src.lds + TILE + (i * NW + wave) * 1024);
    }
  };
  auto issue_kv = [&](int j, int stage) {
    const KvSrc src = kv_src(j, stage);
    static_for<2 * Tile::INST>([&](auto I_) { kv_load(I_, src); });
  };

  // per-lane LDS addresses of the fragment reads, one register per k-step (row-wise) and per (column block, half)
  // (transposed); stage, tile and sub-row offsets ride in the instructions' immediates, so the loop has no address
  // arithmetic at all (computed per read they were 150 of the loop's 355 vector instructions per step).  With
  // 512-byte rows (head_dim 256) the registers are not there and a stage no longer fits the 16-bit immediate: that
  // width computes its addresses per read.
  const RowRead<RB> rr(l32, g);
  const TrRead<RB> tt(i16, q4);
  constexpr bool kPre = D <= 128;
  unsigned ra[kPre ? KSQ : 1], ta[kPre ? DT : 1][2];
  if constexpr (kPre) {
#pragma unroll
    for (int ks = 0; ks < KSQ; ks++) ra[ks] = lds_base + rr.rowb + (rr.xk ^ (ks * 32));
#pragma unroll
    for (int c = 0; c < DT; c++)
#pragma unroll
      for (int h2 = 0; h2 < 2; h2++) ta[c][h2] = lds_base + (tt.tl ^ ((c << 6) | (h2 << 5)));
  }

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

  // One K/V step on LDS stage STAGE; MASKED: the step meets the causal diagonal of this wave's rows.
  // One wave per SIMD (the kernel's registers allow no second), so whatever
  // is to overlap the MFMAs stands between them in this wave's own instruction stream:
  //   phase 1   S^T, dP^T of key tile 0         | the loads of the next step's tiles, one behind each k-step's first MFMA
  //   phase 2   S^T, dP^T of key tile 1         | the softmax / dS arithmetic of key tile 0; the first K^T fragments
  //   phase 3   dQ^T += K^T dS^T, key tile 0    | the softmax / dS arithmetic of key tile 1
  //   phase 4   dQ^T += K^T dS^T, key tile 1
  // (Measured on the kernel's cycle counter before: 16 MFMAs 500 cycles, the arithmetic of a key tile 527 cycles with
  // no MFMA in flight, the eight loads as a burst 323, the step 3283 for 1536 cycles of MFMAs.)
  // The arithmetic of a key tile is a list of independent operations, stage after stage over its 16 elements per
  // lane - u = dP - delta, t = S * scale - M, p = 2^t, (mask,) dS = p * u, conversions in pairs -, of which each
  // MFMA slot takes a slice: an operation and the one that needs its result are then 16 operations apart.
  auto step = [&](const int j, auto STAGE_, auto MASKED_) {
    constexpr int stage = decltype(STAGE_)::value;
    constexpr bool masked = decltype(MASKED_)::value;
    constexpr int KOFF = kPre ? stage * 2 * TILE : 0, VOFF = KOFF + TILE;
    const unsigned sbase = kPre ? 0u : lds_base + (unsigned)(stage * 2 * TILE);
    auto row_addr = [&](auto KS_) {
      constexpr int ks = decltype(KS_)::value;
      if constexpr (kPre) return ra[ks];
      else return rr.template addr<ks>(sbase);
    };
    auto tr_addr = [&](auto C_, auto H_) {
      constexpr int c = decltype(C_)::value, h2 = decltype(H_)::value;
      if constexpr (kPre) return ta[c][h2];
      else return tt.template addr<c, h2>(sbase);
    };
    using I0 = std::integral_constant<int, 0>; using I1 = std::integral_constant<int, 1>;
    // (behind the last step its own tiles once more, into the stage nobody reads: no branch around the loads, whose
    // join the register allocator could use to copy fragment registers with reads still in flight)
    const KvSrc nsrc = kv_src(min(j + 1, nsteps - 1), stage ^ 1);
    V8 dsf[QT][4];
    f32x16 s[2][QT], dp[2][QT];
    i32x4 kf[2], vf[2];
    i32x2 tf[2][DT][2];
    constexpr int NOPS = 16 * (masked ? 5 : 4) + 8;   // operations of a key tile's arithmetic
    auto softmax_ops = [&](auto A_, auto FROM_, auto N_) {
      constexpr int a = decltype(A_)::value;
      static_for<decltype(N_)::value>([&](auto O_) {
        constexpr int i = decltype(FROM_)::value + decltype(O_)::value;
        if constexpr (i < NOPS) {
          constexpr int st = i / 16, r = i % 16;
          constexpr int kind = (!masked && st >= 3) ? st + 1 : st;   // 0 u, 1 t, 2 p, 3 mask, 4 dS, 5 conversions
#pragma unroll
          for (int b = 0; b < QT; b++) {
            if constexpr (kind == 0) dp[a][b][r] -= d_row[b];
            else if constexpr (kind == 1) s[a][b][r] = fmaf(s[a][b][r], qk_scale, -m_row[b]);
            else if constexpr (kind == 2) s[a][b][r] = fast_exp2(s[a][b][r]);
            else if constexpr (kind == 3) {
              const int kv = j * BN + a * 32 + (r >> 2) * 8 + g * 4 + (r & 3);
              if (kv > row0 + b * 32 + l32) s[a][b][r] = 0.f;
            } else if constexpr (kind == 4) dp[a][b][r] *= s[a][b][r];
            else if constexpr (r < 8) {   // elements 2 r, 2 r + 1
              dsf[b][a * 2 + (r >> 2)][(2 * r) & 7] = (S)dp[a][b][2 * r];
              dsf[b][a * 2 + (r >> 2)][(2 * r + 1) & 7] = (S)dp[a][b][2 * r + 1];
            }
          }
        }
      });
    };
    auto read_t = [&](auto T_, auto C_, i32x2 (&dst)[DT][2]) {   // the two halves of K^T fragment (t, c)
      constexpr int t = decltype(T_)::value, c = decltype(C_)::value;
      dst[c][0] = lds_read_tr16_b64<KOFF + 16 * t * RB>(tr_addr(C_, I0{}));
      dst[c][1] = lds_read_tr16_b64<KOFF + (16 * t + 8) * RB>(tr_addr(C_, I1{}));
    };
    // (the padded forms guard every load with a per-lane test - control flow, at whose joins the register allocator
    // may copy registers: their loads go first, while no fragment read is in flight)
    if constexpr (PAD) static_for<2 * Tile::INST>([&](auto I_) { kv_load(I_, nsrc); });
    // ---- phases 1 and 2: S^T and dP^T of key tile a
    kf[0] = lds_read_b128<KOFF>(row_addr(I0{}));
    vf[0] = lds_read_b128<VOFF>(row_addr(I0{}));
    static_for<2>([&](auto A_) {
      constexpr int a = decltype(A_)::value;
      constexpr int XPS = (NOPS + 2 * KSQ - 1) / (2 * KSQ);   // operations per MFMA slot of phase 2
      static_for<KSQ>([&](auto KS_) {
        constexpr int ks = decltype(KS_)::value;
        constexpr int cur = ks & 1, nxt = cur ^ 1;
        // the reads of the k-step to come; in phase 2's last two k-steps the first K^T fragments instead / as well
        constexpr int late = (a == 1 && ks >= KSQ - 2) ? DT * (ks - (KSQ - 2) + 0) : 0;   // K^T reads issued before this k-step
        if constexpr (ks + 1 < KSQ) {
          kf[nxt] = lds_read_b128<KOFF + a * 32 * RB>(row_addr(std::integral_constant<int, ks + 1 < KSQ ? ks + 1 : 0>{}));
          vf[nxt] = lds_read_b128<VOFF + a * 32 * RB>(row_addr(std::integral_constant<int, ks + 1 < KSQ ? ks + 1 : 0>{}));
          lds_wait<2 + late>();
        } else if constexpr (a == 0) {
          // (the first fragments of key tile 1, so that phase 2 starts with its operands on the way)
          kf[nxt] = lds_read_b128<KOFF + 32 * RB>(row_addr(I0{}));
          vf[nxt] = lds_read_b128<VOFF + 32 * RB>(row_addr(I0{}));
          lds_wait<2>();
        } else {
          lds_wait<late>();
        }
        lds_use(kf[cur]);
        lds_use(vf[cur]);
#pragma unroll
        for (int b = 0; b < QT; b++)
          s[a][b] = mfma32(__builtin_bit_cast(V8, kf[cur]), qf[b][ks], ks == 0 ? f32x16{} : s[a][b]);
        if constexpr (a == 0) {
          if constexpr (!PAD && 2 * ks < 2 * Tile::INST) kv_load(std::integral_constant<int, 2 * ks < 2 * Tile::INST ? 2 * ks : 0>{}, nsrc);
        } else {
          softmax_ops(I0{}, std::integral_constant<int, 2 * ks * XPS>{}, std::integral_constant<int, XPS>{});
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int b = 0; b < QT; b++)
          dp[a][b] = mfma32(__builtin_bit_cast(V8, vf[cur]), dof[b][ks], ks == 0 ? f32x16{} : dp[a][b]);
        if constexpr (a == 0) {
          if constexpr (!PAD && 2 * ks + 1 < 2 * Tile::INST) kv_load(std::integral_constant<int, 2 * ks + 1 < 2 * Tile::INST ? 2 * ks + 1 : 0>{}, nsrc);
        } else {
          softmax_ops(I0{}, std::integral_constant<int, (2 * ks + 1) * XPS>{}, std::integral_constant<int, XPS>{});
          if constexpr (ks >= KSQ - 2) {
            // half of the first K^T fragments behind each of the last two k-steps
            static_for<DT / 2>([&](auto C_) { read_t(I0{}, std::integral_constant<int, (ks - (KSQ - 2)) * (DT / 2) + decltype(C_)::value>{}, tf[0]); });
          }
        }
        __builtin_amdgcn_sched_barrier(0);
      });
    });
    // ---- phases 3 and 4: dQ^T += K^T dS^T, [DT d tiles][QT q tiles], 4 k-steps of 16 key rows.  The fragments of
    // k-step t + 1 are requested one behind each MFMA of k-step t, so a fragment is DT MFMAs old when it is used
    // and DT - 1 younger requests may still be outstanding.
    constexpr int XPD = (NOPS + 2 * DT - 1) / (2 * DT);   // operations per MFMA slot of phase 3
    static_for<4>([&](auto T_) {
      constexpr int t = decltype(T_)::value;
      constexpr int cur = t & 1, nxt = cur ^ 1;
      static_for<DT>([&](auto C_) {
        constexpr int c = decltype(C_)::value;
        lds_wait<(t + 1 < 4) ? 2 * (DT - 1) : 2 * (DT - 1 - c)>();
        lds_use(tf[cur][c][0]);
        lds_use(tf[cur][c][1]);
        i32x4 both = __builtin_shufflevector(tf[cur][c][0], tf[cur][c][1], 0, 1, 2, 3);
#pragma unroll
        for (int b = 0; b < QT; b++) dq[c][b] = mfma32(__builtin_bit_cast(V8, both), dsf[b][t], dq[c][b]);
        if constexpr (t + 1 < 4) read_t(std::integral_constant<int, t + 1 < 4 ? t + 1 : 0>{}, C_, tf[nxt]);
        if constexpr (t < 2) softmax_ops(I1{}, std::integral_constant<int, (t * DT + c) * XPD>{}, std::integral_constant<int, XPD>{});
        __builtin_amdgcn_sched_barrier(0);
      });
    });
  };
  auto run = [&](const int j, auto STAGE_, auto MASKED_) {
    if (j <= wave_last && row0 < p.N) step(j, STAGE_, MASKED_);
    else issue_kv(min(j + 1, nsteps - 1), decltype(STAGE_)::value ^ 1);
    wait_all();
    __syncthreads();
  };
  // The steps below the diagonal run in a loop of their own, the few that meet it in a second one: with both
  // forms behind a branch inside one loop the register allocator gave the two bodies different registers for the
  // accumulators and copied all 64 of them back and forth at the join of every step.  (Every wave runs every
  // step's loads and barrier in either loop, so the waves of a workgroup may split at different steps.)
  using I0 = std::integral_constant<int, 0>; using I1 = std::integral_constant<int, 1>;
  const int nplain = min(wave_first_masked, nsteps);
  int j = 0;
  for (; j + 1 < nplain; j += 2) {
    run(j, I0{}, std::false_type{});
    run(j + 1, I1{}, std::false_type{});
  }
  if (j < nplain) { run(j, I0{}, std::false_type{}); j++; }
  for (; j < nsteps; j++) {
    if (j & 1) run(j, I1{}, std::true_type{});
    else run(j, I0{}, std::true_type{});
  }

  // dQ rows through this wave's share of the K/V stages (free: every step ends with a full wait and a barrier)
#pragma unroll
  for (int b = 0; b < QT; b++) {
    const int r0 = row0 + b * 32;
    if (r0 >= p.N) continue;   // (wave-uniform)
    f32x16 t[DT];
#pragma unroll
    for (int c = 0; c < DT; c++) t[c] = dq[c][b];
    store_rows_transposed<S, D, PAD>(t, p.sm_scale, lds_base + (wave * QT + b) * 32 * (D * 2), p.dq + head_off + (int64_t)r0 * pitch,
                                     pitch, p.N - r0, p.d_real, lane);
  }
}

template <typename V8, int D, bool PAD = false>
static int launch_bwd_d(const AttnArgs& p, hipStream_t stream) {
  {
    constexpr int QT = 1, NW = 4, BM = NW * QT * 32;
    constexpr int smem = 2 * 2 * 64 * D * 2;
    static bool attr_set = false;
    if (!attr_set) {
      hipError_t e = hipFuncSetAttribute((const void*)attn_bwd_dq_kernel<V8, D, QT, NW, PAD>,
                                         hipFuncAttributeMaxDynamicSharedMemorySize, smem);
      if (e != hipSuccess) return (int)e;
      attr_set = true;
    }
    int nqb = (p.N + BM - 1) / BM;
    attn_bwd_dq_kernel<V8, D, QT, NW, PAD><<<dim3(nqb * p.Z * p.H), dim3(NW * 64), smem, stream>>>(p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return (int)e;
  }
  return 0;
}

int attn_bwd_dkdv_launch(const AttnArgs& p, bool bf16, hipStream_t stream);  // attn_bwd_dkdv.hip

int attn_bwd_launch(const AttnArgs& p, bool bf16, hipStream_t stream) {
  int rc;
  if (p.d_real < p.D) rc = bf16 ? launch_bwd_d<bf16x8, 64, true>(p, stream) : launch_bwd_d<f16x8, 64, true>(p, stream);
  else if (p.D == 256) rc = bf16 ? launch_bwd_d<bf16x8, 256>(p, stream) : launch_bwd_d<f16x8, 256>(p, stream);
  else if (bf16) rc = p.D == 128 ? launch_bwd_d<bf16x8, 128>(p, stream) : launch_bwd_d<bf16x8, 64>(p, stream);
  else rc = p.D == 128 ? launch_bwd_d<f16x8, 128>(p, stream) : launch_bwd_d<f16x8, 64>(p, stream);
  if (rc) return rc;
  return attn_bwd_dkdv_launch(p, bf16, stream);
}

int attn_bwd_pre_launch(const AttnArgs& p, bool bf16, hipStream_t stream) {
  dim3 grid, block(256);
  if (p.D == 256) {
    grid = dim3((p.N + 7) / 8, p.Z * p.H);
    if (bf16) attn_bwd_pre_kernel<bf16x8, 256><<<grid, block, 0, stream>>>(p);
    else attn_bwd_pre_kernel<f16x8, 256><<<grid, block, 0, stream>>>(p);
  } else if (p.D == 128) {
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

// Fused flash-attention forward for gfx950 (fp16 / bf16, head_dim 64, 128 or 256).
//
// Same algorithm as the reference `_attn_fwd` / `_attn_fwd_inner`
// (python/tutorials/06-fused-attention.py:25-75, :98-187): a Q tile stays resident, K/V stream
// past it in BLOCK_N = 64 steps, online softmax in fp32 in the exp2 domain with
// qk_scale = sm_scale * 1.44269504 (:160-161), P rounded to the input type before the second
// product (:66-70) while the normaliser sums the unrounded P (:57-58), causal blocks above the
// diagonal are skipped and only the diagonal block is masked (:33-40, :49-53), and
// M = m + log2(l), O = acc / l at the end (:183-187).
//
// MI355X-first layout of the work:
//   * every wave owns QT*32 query rows and all of head_dim; the score tile is computed
//     TRANSPOSED (S^T = K Q^T), so a lane holds 16 scores of ONE query row per 32x32 MFMA tile:
//     row max / row sum are in-lane reductions plus one 32-lane swap, the rescale factor is a
//     per-lane scalar, and the fp32 -> 16-bit P^T registers are already the B operand of the
//     second MFMA (O^T = V^T P^T) - P never goes through LDS;
//   * K and V tiles go global -> LDS by direct 16-byte loads into two stages; K rows are read
//     back as MFMA A operands with ds_read_b128, V is transposed on the fly by
//     ds_read_b64_tr_b16; one XOR swizzle (attn_tiles.h) keeps both conflict free;
//   * heads are laid out over XCDs so that the query blocks sharing one K/V stay on one L2,
//     and causal query blocks are issued longest-first.
#include "attn_tiles.h"
#include "launch.h"

#ifndef MI355_ATTN_K_AHEAD
#define MI355_ATTN_K_AHEAD 1
#endif
#ifndef MI355_ATTN_V_EARLY
#define MI355_ATTN_V_EARLY 1
#endif

namespace mi355 {

template <typename V8> struct Elem;
template <> struct Elem<bf16x8> { using type = __bf16; };
template <> struct Elem<f16x8> { using type = _Float16; };

// PAD (D = 64 only): the tensors hold p.d_real = 16 or 32 columns per row; the missing columns are zeros that
// never exist in memory - fragments loaded straight into registers are zero-filled, the K / V tiles in LDS are
// zeroed once and only the chunks present are ever loaded, and only the first d_real columns of O are stored.
// Scores, softmax and those columns of O are what a HEAD_DIM d_real kernel computes (zero columns add nothing).
template <typename V8, int D, int QT, int NW, bool PAD = false>
__global__ __launch_bounds__(NW * 64, 1) void attn_fwd_kernel(AttnArgs p) {
  using S = typename Elem<V8>::type;
  constexpr int BM = NW * QT * 32, BN = 64;
  constexpr int RB = D * 2;            // bytes per K/V row
  using Tile = AttnTile<RB, BN, NW>;
  constexpr int TILE = Tile::BYTES;    // bytes of one K or V tile
  constexpr int INST = Tile::INST;     // direct-load instructions per wave and tile
  constexpr int KSQ = D / 16;          // MFMA k-steps of S^T = K Q^T
  constexpr int DT = D / 32;           // 32-row tiles of O^T

  extern __shared__ __attribute__((aligned(1024))) char smem[];
  LDS_PTR(char) const lds = (LDS_PTR(char))smem;  // [stage][K tile | V tile]

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, g = lane >> 5, i16 = lane & 15, q4 = lane >> 4;

  // block -> (head, query block): consecutive logical ids (same XCD) walk the query blocks of
  // one head; causal blocks in descending order of work
  const int nqb = (p.N + BM - 1) / BM;
  int pid = xcd_remap(blockIdx.x, nqb * p.Z * p.H);
  const int hz = pid / nqb;
  int qb = pid % nqb;
  if (p.causal) qb = nqb - 1 - qb;
  const int z = hz / p.H, h = hz % p.H;
  const int m0 = qb * BM;
  const int row0 = m0 + wave * QT * 32;  // first query row of this wave

  const char* qbase = p.q + ((int64_t)z * p.sq[0] + (int64_t)h * p.sq[1]) * 2;
  const char* kbase = p.k + ((int64_t)z * p.sk[0] + (int64_t)h * p.sk[1]) * 2;
  const char* vbase = p.v + ((int64_t)z * p.sv[0] + (int64_t)h * p.sv[1]) * 2;
  char* obase = p.o + ((int64_t)z * p.so[0] + (int64_t)h * p.so[1]) * 2;
  const int64_t qpitch = p.sq[2] * 2, kpitch = p.sk[2] * 2, vpitch = p.sv[2] * 2, opitch = p.so[2] * 2;

  // ---- Q fragments (B operand of S^T): lane (row l32, half g) holds Q[row][16*ks + 8*g .. +8]
  V8 qf[QT][KSQ];
#pragma unroll
  for (int b = 0; b < QT; b++) {
    int r = min(row0 + b * 32 + l32, p.N - 1);
    const char* src = qbase + (int64_t)r * qpitch + g * 16;
#pragma unroll
    for (int ks = 0; ks < KSQ; ks++) {
      if (!PAD || ks * 32 + g * 16 < p.d_real * 2) qf[b][ks] = *(const V8*)(src + ks * 32);
      else qf[b][ks] = V8{};
    }
  }

  // ---- direct global -> LDS copies of the K and V tiles: a scalar tile base that advances with
  // the step plus a 32-bit per-lane offset (64 rows of K or V span less than 2^31 bytes, which the
  // host checks), so a load costs no vector arithmetic
  unsigned offK[INST], offV[INST];
  bool present[INST];
#pragma unroll
  for (int i = 0; i < INST; i++) {
    offK[i] = (unsigned)Tile::off(kpitch, wave, lane, i);
    offV[i] = (unsigned)Tile::off(vpitch, wave, lane, i);
    present[i] = !PAD || Tile::chunk_present(wave, lane, i, p.d_real * 2);
  }
  const unsigned lds_base = lds_addr(lds);
  if constexpr (PAD) {
    lds_zero(lds, 2 * 2 * TILE, tid, NW * 64);
    __syncthreads();
  }
  auto issue_kv = [&](int j, int stage) {
    const unsigned kd = lds_base + stage * (2 * TILE), vd = kd + TILE;
    const char* ksrc = kbase + (int64_t)j * BN * kpitch;
    const char* vsrc = vbase + (int64_t)j * BN * vpitch;
#pragma unroll
    for (int i = 0; i < INST; i++) {
      if (present[i]) {
        async_copy16_sbase(ksrc, offK[i], kd + (i * NW + wave) * 1024);
        async_copy16_sbase(vsrc, offV[i], vd + (i * NW + wave) * 1024);
      }
    }
  };

  // ---- per-lane LDS addresses (row-wise K operand, transposed V operand), one register per
  // k-step / column block; stage and sub-tile offsets go into the instructions' immediates
  const RowRead<RB> rk(l32, g);
  const TrRead<RB> tv(i16, q4);
  const unsigned lds0 = lds_addr(lds);
  unsigned ka[KSQ], va[DT][2];
#pragma unroll
  for (int ks = 0; ks < KSQ; ks++) ka[ks] = lds0 + rk.rowb + (rk.xk ^ (ks * 32));
#pragma unroll
  for (int c = 0; c < DT; c++)
#pragma unroll
    for (int h2 = 0; h2 < 2; h2++) va[c][h2] = lds0 + (tv.tl ^ ((c << 6) | (h2 << 5)));

  f32x16 oacc[DT][QT];
#pragma unroll
  for (int c = 0; c < DT; c++)
#pragma unroll
    for (int b = 0; b < QT; b++)
#pragma unroll
      for (int r = 0; r < 16; r++) oacc[c][b][r] = 0.f;
  float m_i[QT], l_i[QT];
#pragma unroll
  for (int b = 0; b < QT; b++) { m_i[b] = -INFINITY; l_i[b] = 0.f; }

  const float qk_scale = p.sm_scale * 1.44269504f;
  // The running maximum only has to bound the scores loosely: it is raised (and the
  // accumulators rescaled) when some row of the wave outgrows it by more than 2^RESCALE_LOG2,
  // so P stays below 2^RESCALE_LOG2 and the result O = acc / l, M = m + log2(l) is unchanged.
  constexpr float RESCALE_LOG2 = 8.f;

  // number of K/V steps of this block / wave
  const int kv_end_blk = p.causal ? min(p.N, m0 + BM) : p.N;
  const int nsteps = (kv_end_blk + BN - 1) / BN;
  const int wave_last = p.causal ? (row0 + QT * 32 - 1) / BN : nsteps - 1;  // last step with unmasked columns
  const int wave_first_masked = p.causal ? row0 / BN : nsteps;              // first step that needs the mask

  issue_kv(0, 0);
  wait_all();
  __syncthreads();

  auto step = [&](const int j, auto STAGE_) {
    constexpr int stage = decltype(STAGE_)::value;
    // the stage offset rides in the instructions' 16-bit immediates where two stages fit below 64 KiB;
    // with 512-byte rows (head_dim 256) a stage is 64 KiB and its offset is added to the addresses
    constexpr bool kStageImm = 2 * 2 * TILE <= 65536;
    constexpr int KOFF = kStageImm ? stage * 2 * TILE : 0, VOFF = KOFF + TILE;
    const unsigned sreg = kStageImm ? 0u : (unsigned)(stage * 2 * TILE);
    if (j + 1 < nsteps) issue_kv(j + 1, stage ^ 1);
    if (j <= wave_last && row0 < p.N) {
      // ---- S^T = K Q^T : [2 kv tiles][QT q tiles]
      f32x16 s[2][QT];
#pragma unroll
      for (int a = 0; a < 2; a++)
#pragma unroll
        for (int b = 0; b < QT; b++)
#pragma unroll
          for (int r = 0; r < 16; r++) s[a][b][r] = 0.f;
      {
        // K fragments KAHEAD k-steps ahead of their MFMAs (KAHEAD + 1 register sets).  Measured: one, two or three
        // k-steps ahead run the same - what the K reads cost (15 % of the kernel in a knock-out) is not their latency
        constexpr int KAHEAD = MI355_ATTN_K_AHEAD;
        i32x4 kf[KAHEAD + 1][2];
        static_for<KAHEAD>([&](auto I_) {
          constexpr int i = decltype(I_)::value;
          if constexpr (i < KSQ) {
            kf[i][0] = lds_read_b128<KOFF>(ka[i] + sreg);
            kf[i][1] = lds_read_b128<KOFF + 32 * RB>(ka[i] + sreg);
          }
        });
        static_for<KSQ>([&](auto KS_) {
          constexpr int ks = decltype(KS_)::value;
          constexpr int cur = ks % (KAHEAD + 1), nxt = (ks + KAHEAD) % (KAHEAD + 1);
          if constexpr (ks + KAHEAD < KSQ) {
            kf[nxt][0] = lds_read_b128<KOFF>(ka[ks + KAHEAD < KSQ ? ks + KAHEAD : 0] + sreg);
            kf[nxt][1] = lds_read_b128<KOFF + 32 * RB>(ka[ks + KAHEAD < KSQ ? ks + KAHEAD : 0] + sreg);
          }
          // reads issued behind those of k-step ks: two per k-step still to come, at most KAHEAD of them
          constexpr int behind = (KSQ - 1 - ks) < KAHEAD ? (KSQ - 1 - ks) : KAHEAD;
          lds_wait<2 * behind>();
          lds_use(kf[cur][0]);
          lds_use(kf[cur][1]);
#pragma unroll
          for (int a = 0; a < 2; a++)
#pragma unroll
            for (int b = 0; b < QT; b++)
              s[a][b] = mfma32(__builtin_bit_cast(V8, kf[cur][a]), qf[b][ks], s[a][b]);
        });
      }
      // (the first V fragments are requested here already: their latency passes behind the softmax arithmetic)
      i32x2 vf[2][DT][2];
      auto read_v = [&](auto T_, i32x2 (&dst)[DT][2]) {
        constexpr int t = decltype(T_)::value;
        static_for<DT>([&](auto C_) {
          constexpr int c = decltype(C_)::value;
          dst[c][0] = lds_read_tr16_b64<VOFF + 16 * t * RB>(va[c][0] + sreg);
          dst[c][1] = lds_read_tr16_b64<VOFF + (16 * t + 8) * RB>(va[c][1] + sreg);
        });
      };
      if constexpr (MI355_ATTN_V_EARLY) read_v(std::integral_constant<int, 0>{}, vf[0]);
      // ---- online softmax, one query row per lane (pair of lanes l, l+32 shares a row)
      V8 pf[QT][4];  // P^T as B operand of the second product, per 16-column k-step
#pragma unroll
      for (int b = 0; b < QT; b++) {
        if (j >= wave_first_masked) {
          const int qrow = row0 + b * 32 + l32;
#pragma unroll
          for (int a = 0; a < 2; a++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
              int kv = j * BN + a * 32 + (r >> 2) * 8 + g * 4 + (r & 3);
              if (kv > qrow) s[a][b][r] = -INFINITY;
            }
        }
        float mx = s[0][b][0];
#pragma unroll
        for (int a = 0; a < 2; a++)
#pragma unroll
          for (int r = 0; r < 16; r++) mx = fmaxf(mx, s[a][b][r]);
        mx = pair_max(mx);
        const float m_new = fmaxf(m_i[b], mx * qk_scale);
        if (__builtin_amdgcn_ballot_w64(m_new > m_i[b] + RESCALE_LOG2) != 0) {
          const float alpha = fast_exp2(m_i[b] - m_new);
          l_i[b] *= alpha;
          m_i[b] = m_new;
#pragma unroll
          for (int c = 0; c < DT; c++)
#pragma unroll
            for (int r = 0; r < 16; r++) oacc[c][b][r] *= alpha;
        }
        const float m_cur = m_i[b];
        float rs = 0.f;
#pragma unroll
        for (int a = 0; a < 2; a++)
#pragma unroll
          for (int r = 0; r < 16; r++) {
            float pv = fast_exp2(fmaf(s[a][b][r], qk_scale, -m_cur));
            s[a][b][r] = pv;
            rs += pv;
          }
        l_i[b] += rs;
        // k-step t = 2a + u covers columns 16t .. 16t+15: registers 8u .. 8u+7 of tile a
#pragma unroll
        for (int t = 0; t < 4; t++)
#pragma unroll
          for (int e = 0; e < 8; e++) pf[b][t][e] = (S)s[t >> 1][b][(t & 1) * 8 + e];
      }
      // ---- O^T += V^T P^T : [DT d tiles][QT q tiles], 4 k-steps of 16 columns
      {
        if constexpr (!MI355_ATTN_V_EARLY) read_v(std::integral_constant<int, 0>{}, vf[0]);
        static_for<4>([&](auto T_) {
          constexpr int t = decltype(T_)::value;
          constexpr int cur = t & 1, nxt = cur ^ 1;
          if constexpr (t + 1 < 4) {
            read_v(std::integral_constant<int, t + 1>{}, vf[nxt]);
            lds_wait<2 * DT>();
          } else {
            lds_wait<0>();
          }
#pragma unroll
          for (int c = 0; c < DT; c++) {
            lds_use(vf[cur][c][0]);
            lds_use(vf[cur][c][1]);
            i32x4 both = __builtin_shufflevector(vf[cur][c][0], vf[cur][c][1], 0, 1, 2, 3);
#pragma unroll
            for (int b = 0; b < QT; b++) oacc[c][b] = mfma32(__builtin_bit_cast(V8, both), pf[b][t], oacc[c][b]);
          }
        });
      }
    }
    wait_all();
    __syncthreads();
  };

  for (int j = 0; j < nsteps; j += 2) {
    step(j, std::integral_constant<int, 0>{});
    if (j + 1 < nsteps) step(j + 1, std::integral_constant<int, 1>{});
  }

  // ---- epilogue: O = acc / l, M = m + log2(l)
#pragma unroll
  for (int b = 0; b < QT; b++) {
    float l = l_i[b];
    l = pair_sum(l);
    const int row = row0 + b * 32 + l32;
    if (row0 + b * 32 >= p.N) continue;   // (wave-uniform: N is a multiple of 32)
    const float inv = 1.f / l;
    if (g == 0 && row < p.N) p.lse[(int64_t)hz * p.N + row] = m_i[b] + log2f(l);
    // (the K/V stages are free: the last step requested nothing and ended with a barrier)
    f32x16 ob[DT];
#pragma unroll
    for (int c = 0; c < DT; c++) ob[c] = oacc[c][b];
    store_rows_transposed<S, D, PAD>(ob, inv, lds0 + (wave * QT + b) * 32 * RB, obase + (int64_t)(row0 + b * 32) * opitch, opitch,
                            p.N - (row0 + b * 32), p.d_real, lane);
  }
}

// ---------------------------------------------------------------------------------------------
// Persistent form: gridDim.x workgroups each walk several (head, query block) items as ONE stream
// of K/V steps.  The direct loads of the next item's first K/V tile are issued during the last
// step of the current one and its Q fragments a whole item ahead, so the per-item start-up (a
// memory round trip for Q and for the first tile, worth about three K/V steps) is hidden.
// Items are dealt round-robin in an order that keeps the workgroups of one XCD on one head; under
// the causal mask odd rounds walk the query blocks short-to-long and even rounds long-to-short, so
// every workgroup gets the same amount of work over two rounds.  One query tile (32 rows) per wave.
// ---------------------------------------------------------------------------------------------
template <typename V8, int D, int NW, bool PAD = false>   // PAD: as in attn_fwd_kernel
__global__ __launch_bounds__(NW * 64, NW == 4 ? 2 : 1) void attn_fwd_stream_kernel(AttnArgs p) {
  using S = typename Elem<V8>::type;
  constexpr int BM = NW * 32, BN = 64;
  constexpr int RB = D * 2;
  using Tile = AttnTile<RB, BN, NW>;
  constexpr int TILE = Tile::BYTES;
  constexpr int INST = Tile::INST;
  constexpr int KSQ = D / 16;
  constexpr int DT = D / 32;

  extern __shared__ __attribute__((aligned(1024))) char smem[];
  LDS_PTR(char) const lds = (LDS_PTR(char))smem;  // [stage][K tile | V tile]

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, g = lane >> 5, i16 = lane & 15, q4 = lane >> 4;

  const int nqb = (p.N + BM - 1) / BM;
  const int total = nqb * p.Z * p.H;
  const int G = gridDim.x;
  const int lid = xcd_remap(blockIdx.x, G);
  const int nitems = (total - lid + G - 1) / G;  // the host keeps G <= total
  const int heads_per_round = max(1, G / nqb);
  const int64_t qpitch = p.sq[2] * 2, kpitch = p.sk[2] * 2, vpitch = p.sv[2] * 2, opitch = p.so[2] * 2;

  // item r of this workgroup -> (head, query block)
  auto item_of = [&](int r, int& hz, int& qb) {
    const int L = r * G + lid;
    hz = L / nqb;
    const int j = L % nqb;
    // direction by the round a head falls into (G / nqb heads per round): a bijection whatever G is,
    // and equal to "even rounds long-to-short" when G is a multiple of nqb
    qb = (p.causal && ((hz / heads_per_round) & 1) == 0) ? nqb - 1 - j : j;
  };
  auto steps_of = [&](int qb) {
    const int kv_end = p.causal ? min(p.N, (qb + 1) * BM) : p.N;
    return (kv_end + BN - 1) / BN;
  };
  auto head_ptr = [&](const char* base, const int64_t* st, int hz) {
    return base + ((int64_t)(hz / p.H) * st[0] + (int64_t)(hz % p.H) * st[1]) * 2;
  };
  auto load_q = [&](V8 (&dst)[KSQ], int hz, int qb) {
    const int r = min(qb * BM + wave * 32 + l32, p.N - 1);
    const char* src = head_ptr(p.q, p.sq, hz) + (int64_t)r * qpitch + g * 16;
#pragma unroll
    for (int ks = 0; ks < KSQ; ks++) {
      if (!PAD || ks * 32 + g * 16 < p.d_real * 2) dst[ks] = *(const V8*)(src + ks * 32);
      else dst[ks] = V8{};
    }
  };

  // ---- state of the item being multiplied
  int c_item = 0, c_hz, c_qb, cj = 0;
  item_of(0, c_hz, c_qb);
  int nsteps = steps_of(c_qb);
  int row0 = c_qb * BM + wave * 32;
  int wave_last = p.causal ? (row0 + 31) / BN : nsteps - 1;
  int wave_first_masked = p.causal ? row0 / BN : nsteps;
  V8 qf[KSQ], qnext[KSQ];
  load_q(qf, c_hz, c_qb);
  {
    int nhz, nqbk;
    item_of(min(1, nitems - 1), nhz, nqbk);
    load_q(qnext, nhz, nqbk);
  }

  // ---- fill cursor: the (item, K/V step) the next direct loads fetch; stops after the last one
  int f_item = 0, fj = 0, f_steps = nsteps;
  const char* f_k = head_ptr(p.k, p.sk, c_hz);
  const char* f_v = head_ptr(p.v, p.sv, c_hz);
  bool f_valid = true;
  unsigned offK[INST], offV[INST];
  bool present[INST];
#pragma unroll
  for (int i = 0; i < INST; i++) {
    offK[i] = (unsigned)Tile::off(kpitch, wave, lane, i);
    offV[i] = (unsigned)Tile::off(vpitch, wave, lane, i);
    present[i] = !PAD || Tile::chunk_present(wave, lane, i, p.d_real * 2);
  }
  const unsigned lds_base = lds_addr(lds);
  if constexpr (PAD) {
    lds_zero(lds, 2 * 2 * TILE, tid, NW * 64);
    __syncthreads();
  }
  // (f_k / f_v point at the tile to fetch and move on by one tile per step: two scalar additions instead of the
  // 64-bit products of a step number - the bookkeeping of this function stands in front of every step's MFMAs)
  const int64_t kstep = (int64_t)BN * kpitch, vstep = (int64_t)BN * vpitch;
  auto issue_fill = [&](int stage) {
    if (!f_valid) return;
    const unsigned kd = lds_base + stage * (2 * TILE), vd = kd + TILE;
    const char* ksrc = f_k;
    const char* vsrc = f_v;
#pragma unroll
    for (int i = 0; i < INST; i++) {
      if (present[i]) {
        async_copy16_sbase(ksrc, offK[i], kd + (i * NW + wave) * 1024);
        async_copy16_sbase(vsrc, offV[i], vd + (i * NW + wave) * 1024);
      }
    }
    f_k += kstep;
    f_v += vstep;
    if (++fj == f_steps) {
      fj = 0;
      if (++f_item < nitems) {
        int hz, qb;
        item_of(f_item, hz, qb);
        f_steps = steps_of(qb);
        f_k = head_ptr(p.k, p.sk, hz);
        f_v = head_ptr(p.v, p.sv, hz);
      } else {
        f_valid = false;
      }
    }
  };

  const RowRead<RB> rk(l32, g);
  const TrRead<RB> tv(i16, q4);
  unsigned ka[KSQ], va[DT][2];
#pragma unroll
  for (int ks = 0; ks < KSQ; ks++) ka[ks] = lds_base + rk.rowb + (rk.xk ^ (ks * 32));
#pragma unroll
  for (int c = 0; c < DT; c++)
#pragma unroll
    for (int h2 = 0; h2 < 2; h2++) va[c][h2] = lds_base + (tv.tl ^ ((c << 6) | (h2 << 5)));

  f32x16 oacc[DT];
#pragma unroll
  for (int c = 0; c < DT; c++)
#pragma unroll
    for (int r = 0; r < 16; r++) oacc[c][r] = 0.f;
  float m_i = -INFINITY, l_i = 0.f;
  const float qk_scale = p.sm_scale * 1.44269504f;
  constexpr float RESCALE_LOG2 = 8.f;  // lazy running maximum, as in attn_fwd_kernel

  issue_fill(0);
  wait_all();
  __syncthreads();

  // one K/V step of the stream in ring stage STAGE; false once the last item is stored
  auto step = [&](auto STAGE_) -> bool {
    constexpr int stage = decltype(STAGE_)::value;
    constexpr int KOFF = stage * 2 * TILE, VOFF = KOFF + TILE;
    const int j = cj;
    issue_fill(stage ^ 1);
    if (j <= wave_last && row0 < p.N) {
      f32x16 s[2];
#pragma unroll
      for (int a = 0; a < 2; a++)
#pragma unroll
        for (int r = 0; r < 16; r++) s[a][r] = 0.f;
      {
        i32x4 kf[2][2];
        kf[0][0] = lds_read_b128<KOFF>(ka[0]);
        kf[0][1] = lds_read_b128<KOFF + 32 * RB>(ka[0]);
        static_for<KSQ>([&](auto KS_) {
          constexpr int ks = decltype(KS_)::value;
          constexpr int cur = ks & 1, nxt = cur ^ 1;
          if constexpr (ks + 1 < KSQ) {
            kf[nxt][0] = lds_read_b128<KOFF>(ka[ks + 1]);
            kf[nxt][1] = lds_read_b128<KOFF + 32 * RB>(ka[ks + 1]);
            lds_wait<2>();
          } else {
            lds_wait<0>();
          }
          lds_use(kf[cur][0]);
          lds_use(kf[cur][1]);
#pragma unroll
          for (int a = 0; a < 2; a++) s[a] = mfma32(__builtin_bit_cast(V8, kf[cur][a]), qf[ks], s[a]);
        });
      }
      V8 pf[4];
      {
        if (j >= wave_first_masked) {
          const int qrow = row0 + l32;
#pragma unroll
          for (int a = 0; a < 2; a++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
              int kv = j * BN + a * 32 + (r >> 2) * 8 + g * 4 + (r & 3);
              if (kv > qrow) s[a][r] = -INFINITY;
            }
        }
        float mx = s[0][0];
#pragma unroll
        for (int a = 0; a < 2; a++)
#pragma unroll
          for (int r = 0; r < 16; r++) mx = fmaxf(mx, s[a][r]);
        mx = pair_max(mx);
        const float m_new = fmaxf(m_i, mx * qk_scale);
        if (__builtin_amdgcn_ballot_w64(m_new > m_i + RESCALE_LOG2) != 0) {
          const float alpha = fast_exp2(m_i - m_new);
          l_i *= alpha;
          m_i = m_new;
#pragma unroll
          for (int c = 0; c < DT; c++)
#pragma unroll
            for (int r = 0; r < 16; r++) oacc[c][r] *= alpha;
        }
        const float m_cur = m_i;
        float rs = 0.f;
#pragma unroll
        for (int a = 0; a < 2; a++)
#pragma unroll
          for (int r = 0; r < 16; r++) {
            float pv = fast_exp2(fmaf(s[a][r], qk_scale, -m_cur));
            s[a][r] = pv;
            rs += pv;
          }
        l_i += rs;
#pragma unroll
        for (int t = 0; t < 4; t++)
#pragma unroll
          for (int e = 0; e < 8; e++) pf[t][e] = (S)s[t >> 1][(t & 1) * 8 + e];
      }
      {
        i32x2 vf[2][DT][2];
        auto read_v = [&](auto T_, i32x2 (&dst)[DT][2]) {
          constexpr int t = decltype(T_)::value;
          static_for<DT>([&](auto C_) {
            constexpr int c = decltype(C_)::value;
            dst[c][0] = lds_read_tr16_b64<VOFF + 16 * t * RB>(va[c][0]);
            dst[c][1] = lds_read_tr16_b64<VOFF + (16 * t + 8) * RB>(va[c][1]);
          });
        };
        read_v(std::integral_constant<int, 0>{}, vf[0]);
        static_for<4>([&](auto T_) {
          constexpr int t = decltype(T_)::value;
          constexpr int cur = t & 1, nxt = cur ^ 1;
          if constexpr (t + 1 < 4) {
            read_v(std::integral_constant<int, t + 1>{}, vf[nxt]);
            lds_wait<2 * DT>();
          } else {
            lds_wait<0>();
          }
#pragma unroll
          for (int c = 0; c < DT; c++) {
            lds_use(vf[cur][c][0]);
            lds_use(vf[cur][c][1]);
            i32x4 both = __builtin_shufflevector(vf[cur][c][0], vf[cur][c][1], 0, 1, 2, 3);
            oacc[c] = mfma32(__builtin_bit_cast(V8, both), pf[t], oacc[c]);
          }
        });
      }
    }
    wait_all();
    __syncthreads();
    if (++cj < nsteps) return true;

    // ---- item finished: O = acc / l, M = m + log2(l); then switch to the next item
    {
      float l = pair_sum(l_i);
      const int row = row0 + l32;
      // (stored from the registers, 16 bytes per lane: register groups 2 a and 2 a + 1 are exchanged between the two
      // lanes of a row first, so that a lane holds 8 consecutive columns - half the requests of 8-byte pieces.  The
      // stores of an item overlap the next item's steps here, and the detour through LDS of attn_fwd_kernel's
      // epilogue measured 0-2 % slower in this kernel.)
      if (row0 < p.N) {   // (wave-uniform: N is a multiple of 32)
        const float inv = 1.f / l;
        if (g == 0) p.lse[(int64_t)c_hz * p.N + row] = m_i + log2f(l);
        char* dst = (char*)head_ptr(p.o, p.so, c_hz) + (int64_t)row * opitch + g * 16;
        typedef __attribute__((ext_vector_type(2))) S S2;
#pragma unroll
        for (int c = 0; c < DT; c++)
#pragma unroll
          for (int a = 0; a < 2; a++) {
            int x0 = __builtin_bit_cast(int, S2{(S)(oacc[c][a * 8] * inv), (S)(oacc[c][a * 8 + 1] * inv)});
            int x1 = __builtin_bit_cast(int, S2{(S)(oacc[c][a * 8 + 2] * inv), (S)(oacc[c][a * 8 + 3] * inv)});
            int y0 = __builtin_bit_cast(int, S2{(S)(oacc[c][a * 8 + 4] * inv), (S)(oacc[c][a * 8 + 5] * inv)});
            int y1 = __builtin_bit_cast(int, S2{(S)(oacc[c][a * 8 + 6] * inv), (S)(oacc[c][a * 8 + 7] * inv)});
            swap32_regs(x0, y0);
            swap32_regs(x1, y1);
            const int d = c * 32 + a * 16 + g * 8;
            if (!PAD || d < p.d_real) *(i32x4*)(dst + (c * 32 + a * 16) * 2) = i32x4{x0, x1, y0, y1};
          }
      }
    }
    if (++c_item >= nitems) return false;
    item_of(c_item, c_hz, c_qb);
    cj = 0;
    nsteps = steps_of(c_qb);
    row0 = c_qb * BM + wave * 32;
    wave_last = p.causal ? (row0 + 31) / BN : nsteps - 1;
    wave_first_masked = p.causal ? row0 / BN : nsteps;
#pragma unroll
    for (int ks = 0; ks < KSQ; ks++) qf[ks] = qnext[ks];
    {
      int nhz, nqbk;
      item_of(min(c_item + 1, nitems - 1), nhz, nqbk);
      load_q(qnext, nhz, nqbk);
    }
#pragma unroll
    for (int c = 0; c < DT; c++)
#pragma unroll
      for (int r = 0; r < 16; r++) oacc[c][r] = 0.f;
    m_i = -INFINITY;
    l_i = 0.f;
    return true;
  };

  while (true) {
    if (!step(std::integral_constant<int, 0>{})) break;
    if (!step(std::integral_constant<int, 1>{})) break;
  }
  wait_all();
}

template <typename V8, int D, int NW, bool PAD = false>
static int launch_fwd_stream(const AttnArgs& p, hipStream_t stream) {
  constexpr int BM = NW * 32;
  constexpr int smem = 2 * 2 * 64 * D * 2;
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)attn_fwd_stream_kernel<V8, D, NW, PAD>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) return (int)e;
    attr_set = true;
  }
  const int total = ((p.N + BM - 1) / BM) * p.Z * p.H;
  // as many workgroups as are resident at once: two per CU with four waves, one with eight
  int grid = p.num_programs > 0 ? p.num_programs * (NW == 4 ? 2 : 1) : total;
  if (grid > total) grid = total;
  attn_fwd_stream_kernel<V8, D, NW, PAD><<<dim3(grid), dim3(NW * 64), smem, stream>>>(p);
  return (int)hipGetLastError();
}

template <typename V8, int D, int QT, int NW, bool PAD = false>
static int launch_fwd(const AttnArgs& p, hipStream_t stream) {
  constexpr int BM = NW * QT * 32;
  constexpr int smem = 2 * 2 * 64 * D * 2;
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)attn_fwd_kernel<V8, D, QT, NW, PAD>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) return (int)e;
    attr_set = true;
  }
  int nqb = (p.N + BM - 1) / BM;
  attn_fwd_kernel<V8, D, QT, NW, PAD><<<dim3(nqb * p.Z * p.H), dim3(NW * 64), smem, stream>>>(p);
  return (int)hipGetLastError();
}

template <typename V8>
static int launch_fwd_d(const AttnArgs& p, int variant, hipStream_t stream) {
  // head dims 16 / 32: the 64-column kernels in their padding form (eight waves; persistent under the causal mask)
  if (p.d_real < p.D) return p.causal ? launch_fwd_stream<V8, 64, 8, true>(p, stream) : launch_fwd<V8, 64, 1, 8, true>(p, stream);
  if (variant == 3 && p.D != 256) return p.D == 128 ? launch_fwd_stream<V8, 128, 4>(p, stream) : launch_fwd_stream<V8, 64, 4>(p, stream);
  if (variant == 4 && p.D != 256) return p.D == 128 ? launch_fwd_stream<V8, 128, 8>(p, stream) : launch_fwd_stream<V8, 64, 8>(p, stream);
  // head_dim 256: four waves of 32 query rows, one wave per SIMD (the O accumulator alone is 128 registers)
  if (p.D == 256) return launch_fwd<V8, 256, 1, 4>(p, stream);
  if (p.D == 128) {
    if (variant == 2) return launch_fwd<V8, 128, 1, 8>(p, stream);
    return variant == 1 ? launch_fwd<V8, 128, 1, 4>(p, stream) : launch_fwd<V8, 128, 2, 4>(p, stream);
  }
  if (variant == 2) return launch_fwd<V8, 64, 1, 8>(p, stream);
  return variant == 1 ? launch_fwd<V8, 64, 1, 4>(p, stream) : launch_fwd<V8, 64, 2, 4>(p, stream);
}

int attn_fwd_launch(const AttnArgs& p, bool bf16, hipStream_t stream) {
  int variant = p.variant;
  return bf16 ? launch_fwd_d<bf16x8>(p, variant, stream) : launch_fwd_d<f16x8>(p, variant, stream);
}

}  // namespace mi355

// Fused flash-attention forward for gfx950, head_dim 128, software pipelined inside each wave on 16x16x32 MFMAs.
//
// Same algorithm as the reference `_attn_fwd` / `_attn_fwd_inner` (python/tutorials/06-fused-attention.py:25-75,
// :98-187) and as attn_fwd.hip: online softmax in fp32 in the exp2 domain with qk_scale = sm_scale * 1.44269504
// (:160-161), P rounded to the input type before the second product (:66-70) while the normaliser sums the
// unrounded P (:57-58), causal blocks above the diagonal skipped and only the diagonal masked (:33-40, :49-53),
// M = m + log2(l), O = acc / l at the end (:183-187).  What differs is how the work is laid over the machine:
//
//   * a workgroup is four waves, ONE per SIMD, each owning 64 query rows (four 16-row tiles b) and all of head_dim,
//     so a K or V fragment read from LDS feeds four MFMAs - half the LDS bytes per flop of a 32-row wave;
//   * both products are 16x16x32 MFMAs, the shape with the least energy per flop on this power-limited board.
//     Scores are computed transposed (S^T = K Q^T): lane (query l16 = lane % 16, kg = lane / 16) holds the four
//     consecutive keys 16 a + 4 kg .. + 3 of its query for key tile a, and the 16-bit P^T registers are, as they
//     stand, the B operand of O^T += V^T P^T once the V^T fragments are read in the matching key order (keys
//     4 kg .. + 3 of two neighbouring key tiles: two transpose reads).  O^T tile c holds d = 16 c + 4 kg .. + 3;
//   * with one wave per SIMD nothing overlaps for free, so the key loop is a three-stage pipeline over sub-steps
//     u of 32 keys:  phase(u) = [ S(u+1) MFMAs | PV(u-1) MFMAs ] with the softmax arithmetic X(u) and every LDS
//     read and global load threaded between them, two or three vector instructions behind each MFMA.  S and P
//     are double buffered in architectural registers; the O accumulators and the Q fragments live in the
//     accumulation registers, pinned there by issuing every MFMA as inline assembly;
//   * the running maximum is lazy (raised only when a score outgrows it by more than 2^8), and the test for that is
//     per lane against a precomputed threshold - no cross-lane traffic on the hot path.  Raising it is a cold
//     branch at the end of a phase: m and l change at once (X(u+1) uses them), the O accumulators are rescaled one
//     phase later, behind the PV MFMAs that still carry the old scale;
//   * K tiles (64 keys) go through a ring of three LDS stages, V tiles through a ring of four, filled by direct
//     global->LDS loads two to three tiles ahead; one workgroup barrier per 64 keys, placed between the S part and
//     the PV part of the even phases where every fragment read on either side of it is of a tile that landed long ago.
#include "attn_tiles.h"
#include "launch.h"

// Build-time knock-outs for timing experiments (results are wrong with any of them set): 1 = no softmax arithmetic,
// 2 = no maximum check, 4 = no LDS fragment reads, 8 = no global loads, 16 = no MFMAs.
#ifndef MI355_P16_KO
#define MI355_P16_KO 0
#endif

namespace mi355 {

namespace {

// ---- MFMAs as inline assembly (operand register files are fixed by the constraints: v = architectural, a = accumulation)
// (the first k-step of a score tile starts from a bias tile: zeros, or -inf where the causal mask hides a key)
template <bool BF>
__device__ __forceinline__ void mfma16_s_first(f32x4& d, const i32x4& k, const i32x4& q, const f32x4& bias) {
#if MI355_DEVICE_PASS
  if constexpr ((MI355_P16_KO & 16) != 0) { d = bias; return; }
  if constexpr (BF) asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %3" : "=&v"(d) : "v"(k), "a"(q), "v"(bias));
  else asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %3" : "=&v"(d) : "v"(k), "a"(q), "v"(bias));
#endif
}
template <bool BF>
__device__ __forceinline__ void mfma16_s_acc(f32x4& d, const i32x4& k, const i32x4& q) {
#if MI355_DEVICE_PASS
  if constexpr ((MI355_P16_KO & 16) != 0) return;
  if constexpr (BF) asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+v"(d) : "v"(k), "a"(q));
  else asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+v"(d) : "v"(k), "a"(q));
#endif
}
template <bool BF>
__device__ __forceinline__ void mfma16_o(f32x4& d, const i32x4& v, const i32x4& pt) {
#if MI355_DEVICE_PASS
  if constexpr ((MI355_P16_KO & 16) != 0) return;
  if constexpr (BF) asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(d) : "v"(v), "v"(pt));
  else asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(d) : "v"(v), "v"(pt));
#endif
}
// every MFMA issued so far has written its result (16 idle slots), and `x` is read only behind this point
__device__ __forceinline__ void retire_mfmas() {
#if MI355_DEVICE_PASS
  asm volatile("s_nop 15" ::: "memory");
#endif
}
__device__ __forceinline__ void pin_a(f32x4& x) {
#if MI355_DEVICE_PASS
  asm volatile("" : "+a"(x));
#endif
}
__device__ __forceinline__ void pin_v(f32x4& x) {
#if MI355_DEVICE_PASS
  asm volatile("" : "+v"(x));
#endif
}
// Arithmetic on a value that went through one of these (empty, but ordered like every assembly statement) stays
// behind the MFMA in front of it in program order: without them the optimiser gathers the softmax arithmetic of a
// whole phase in front of the phase's first MFMA, where nothing overlaps it.
__device__ __forceinline__ void pin_f(float& x) {
#if MI355_DEVICE_PASS
  asm volatile("" : "+v"(x));
#endif
}
__device__ __forceinline__ void pin_i(int& x) {
#if MI355_DEVICE_PASS
  asm volatile("" : "+v"(x));
#endif
}
// two idle slots: a vector instruction's result may be read by an assembly MFMA behind this
__device__ __forceinline__ void settle_valu() {
#if MI355_DEVICE_PASS
  asm volatile("s_nop 1" ::: "memory");
#endif
}

// Exchange between the 16-lane rows of a wave: fed with two copies of x, v_permlane16_swap leaves
// (row 0, row 0, row 2, row 2) in the first and (row 1, row 1, row 3, row 3) in the second register.
__device__ __forceinline__ void swap16f(float x, float& r0, float& r1) {
  float a = x, b = x;
#if MI355_DEVICE_PASS
  asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(a), "+v"(b));
#endif
  r0 = a;
  r1 = b;
}
// maximum / sum over the four lanes l16 + 16 {0, 1, 2, 3} that share a query row
__device__ __forceinline__ float quad_max(float x) { float a, b; swap16f(x, a, b); return pair_max(fmaxf(a, b)); }
__device__ __forceinline__ float quad_sum(float x) { float a, b; swap16f(x, a, b); return pair_sum(a + b); }

// V tile swizzle: a transpose read is served two 16-lane groups at a time, four consecutive keys each and four
// keys apart, the same 16 columns - the three terms put those 8 x 32 bytes on different banks
__device__ __forceinline__ int vswz16(int row) { return ((row & 3) << 2) | (((row >> 2) & 1) << 1) | ((row >> 3) & 1); }

template <typename S>
__device__ __forceinline__ int pack2(float x, float y) {
  typedef __attribute__((ext_vector_type(2))) S S2;
  return __builtin_bit_cast(int, S2{(S)x, (S)y});
}

}  // namespace

template <typename S, bool BF>
__global__ __launch_bounds__(256, 1) void attn_fwd_p16_kernel(AttnArgs p) {
  constexpr int NW = 4, BM = 256, BN = 64, RB = 256;
  constexpr int TILE = BN * RB;          // 16 KiB per K or V tile
  constexpr int KNS = 3, VNS = 4;        // ring depths
  constexpr int VBASE = KNS * TILE;
  constexpr int INST = TILE / 1024 / NW; // direct loads per wave and tile (4)
  constexpr int GROUP = 2 * INST;        // loads per wave and 64 keys
  constexpr float RESCALE_LOG2 = 8.f;

  extern __shared__ __attribute__((aligned(1024))) char smem[];
  const unsigned lds0 = lds_addr((LDS_PTR(const void))smem);

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l16 = lane & 15, kg = lane >> 4;

  const int nqb = p.N / BM;
  int pid = xcd_remap(blockIdx.x, nqb * p.Z * p.H);
  const int hz = pid / nqb;
  int qb = pid % nqb;
  if (p.causal) qb = nqb - 1 - qb;       // longest first
  const int z = hz / p.H, h = hz % p.H;
  const int m0 = qb * BM;
  const int row0 = m0 + wave * 64;       // first query row of this wave

  const char* qbase = p.q + ((int64_t)z * p.sq[0] + (int64_t)h * p.sq[1]) * 2;
  const char* kbase = p.k + ((int64_t)z * p.sk[0] + (int64_t)h * p.sk[1]) * 2;
  const char* vbase = p.v + ((int64_t)z * p.sv[0] + (int64_t)h * p.sv[1]) * 2;
  char* obase = p.o + ((int64_t)z * p.so[0] + (int64_t)h * p.so[1]) * 2;
  const int64_t qpitch = p.sq[2] * 2, kpitch = p.sk[2] * 2, vpitch = p.sv[2] * 2, opitch = p.so[2] * 2;

  // work of the workgroup and of this wave, in 64-key tiles and 32-key sub-steps
  const int nblocks = p.causal ? (m0 + BM) / BN : p.N / BN;
  const int L = p.causal ? (row0 + 63) / 32 : 2 * nblocks - 1;     // this wave's last sub-step
  const int first_masked = p.causal ? row0 / 32 : 2 * nblocks;     // its first sub-step that meets the diagonal

  // ---- Q fragments (B operand of S^T): lane (query l16 of tile b, kg) holds Q[row][32 ks + 8 kg .. + 8]
  i32x4 qf[4][4];
#pragma unroll
  for (int b = 0; b < 4; b++) {
    const char* src = qbase + (int64_t)(row0 + b * 16 + l16) * qpitch + kg * 16;
#pragma unroll
    for (int ks = 0; ks < 4; ks++) qf[b][ks] = *(const i32x4*)(src + ks * 64);
  }

  // ---- direct loads: instruction i of a wave moves rows 4 (4 i + wave) .. + 3 (lane: row lane / 16, physical
  // chunk lane % 16; it fetches the logical chunk that the swizzle puts there)
  unsigned offK[INST], offV[INST];
#pragma unroll
  for (int i = 0; i < INST; i++) {
    const int r = (i * NW + wave) * 4 + (lane >> 4), pc = lane & 15;
    offK[i] = (unsigned)(r * kpitch) + ((pc ^ tile_swz<RB>(r)) << 4);
    offV[i] = (unsigned)(r * vpitch) + ((pc ^ vswz16(r)) << 4);
  }
  const int64_t kstep = (int64_t)BN * kpitch, vstep = (int64_t)BN * vpitch;
  auto load_k = [&](auto I_, int blk, auto SETTLE_) {      // load I of K tile `blk` (clamped) into its ring slot
    constexpr int i = decltype(I_)::value;
    const int bc = min(blk, nblocks - 1);
    async_copy16_sbase<decltype(SETTLE_)::value>(kbase + bc * kstep, offK[i], lds0 + (blk % KNS) * TILE + (i * NW + wave) * 1024);
  };
  auto load_v = [&](auto I_, int blk, auto SETTLE_) {
    constexpr int i = decltype(I_)::value;
    const int bc = min(blk, nblocks - 1);
    async_copy16_sbase<decltype(SETTLE_)::value>(vbase + bc * vstep, offV[i], lds0 + VBASE + (blk % VNS) * TILE + (i * NW + wave) * 1024);
  };

  // ---- fragment addresses.  K: lane (key l16 of tile a, kg) of k-step ks reads chunk 4 ks + kg of its row:
  // ka ^ (ks << 6).  V: lane i16 of group kg addresses key row 4 kg + i16 / 4 (+ 16 per key tile) and the 8 bytes
  // i16 & 3 of the 32-byte group of d tile c: va ^ (c << 5).  Ring slot offsets are added per 64 keys.
  const unsigned ka = lds0 + l16 * RB + ((((l16 & 3) << 2) | (kg ^ (l16 >> 2))) << 4);
  const int vx = l16 >> 2, ve = (l16 & 3) >> 1;
  const unsigned va = lds0 + VBASE + (4 * kg + vx) * RB + ((((vx << 2) | ((kg & 1) << 1) | (kg >> 1)) ^ ve) << 4) + (l16 & 1) * 8;
  unsigned kad[4], vad[8];           // addresses in the ring slots currently read

  // ---- state
  f32x4 oacc[8][4];                  // O^T tiles [d tile c][query tile b], accumulation registers
#pragma unroll
  for (int c = 0; c < 8; c++)
#pragma unroll
    for (int b = 0; b < 4; b++) oacc[c][b] = f32x4{0.f, 0.f, 0.f, 0.f};
  f32x4 s[2][2][4];                  // S^T [buffer][key tile a][query tile b]
  i32x4 pf[2][4];                    // P^T [buffer][query tile b]: B operand of the second product
#pragma unroll
  for (int b = 0; b < 4; b++) pf[1][b] = i32x4{0, 0, 0, 0};
  i32x4 kf[3];                       // K fragments in flight
  i32x2 vf[3][2];                    // V^T fragments in flight (two transpose reads each)
  float m_i[4], l_i[4], thr[4], pend[4], mxl[4];
#pragma unroll
  for (int b = 0; b < 4; b++) { m_i[b] = -INFINITY; l_i[b] = 0.f; thr[b] = -INFINITY; pend[b] = 1.f; mxl[b] = -INFINITY; }
  unsigned pend_mask = 0;            // query tiles whose O accumulators await a rescale (wave-uniform)
  const float qk_scale = p.sm_scale * 1.44269504f;
  const float inv_scale = 1.f / qk_scale;
  int dlt[4];                        // causal: key 32 u + 16 a + r is masked for this lane when it exceeds dlt[b]
#pragma unroll
  for (int b = 0; b < 4; b++) dlt[b] = row0 + 16 * b + l16 - 4 * kg;
  f32x4 mb[2][4];                    // bias tiles of the scores [key tile a][query tile b]: 0, or -inf where masked
#pragma unroll
  for (int a = 0; a < 2; a++)
#pragma unroll
    for (int b = 0; b < 4; b++) mb[a][b] = f32x4{0.f, 0.f, 0.f, 0.f};

  // ---- pieces of a phase
  // fragment reads: K fragment n = 2 ks + a of the half HK of the current K slot; V fragment c of the half HV
  auto read_k = [&](auto N_, auto HK_, i32x4& dst) {
    constexpr int n = decltype(N_)::value, ks = n >> 1, a = n & 1, hk = decltype(HK_)::value;
    if constexpr ((MI355_P16_KO & 4) == 0) dst = lds_read_b128<hk * 32 * RB + a * 16 * RB>(kad[ks]);
  };
  auto read_v = [&](auto C_, auto HV_, i32x2 (&dst)[2]) {
    constexpr int c = decltype(C_)::value, hv = decltype(HV_)::value;
    if constexpr ((MI355_P16_KO & 4) != 0) return;
    dst[0] = lds_read_tr16_b64<hv * 32 * RB>(vad[c]);
    dst[1] = lds_read_tr16_b64<hv * 32 * RB + 16 * RB>(vad[c]);
  };
  // X: element e = 0 .. 31 of the sub-step whose scores sit in buffer PAR: query tile b = e & 3, index i = e >> 2
  // (key tile a = i >> 2, register r = i & 3); consecutive elements belong to different tiles, so the additions
  // into l_i[b] of neighbouring slices do not wait for one another
  auto x_elem = [&](auto PAR_, auto E_) {
    constexpr int par = decltype(PAR_)::value, e = decltype(E_)::value, b = e & 3, i = e >> 2, a = i >> 2, r = i & 3;
    if constexpr ((MI355_P16_KO & 1) != 0) return;
    pin_v(s[par][a][b]);
    const float pv = fast_exp2(fmaf(s[par][a][b][r], qk_scale, -m_i[b]));
    s[par][a][b][r] = pv;
    l_i[b] += pv;
    pin_f(l_i[b]);
    if constexpr ((r & 1) == 1) {
      int w = pack2<S>(s[par][a][b][r - 1], pv);
      pin_i(w);
      pf[par][b][a * 2 + (r >> 1)] = w;
    }
  };
  // the lane's largest score of query tile b in buffer PAR
  auto check_b = [&](auto PAR_, auto B_) {
    constexpr int par = decltype(PAR_)::value, b = decltype(B_)::value;
    if constexpr ((MI355_P16_KO & 2) != 0) return;
    float mx = fmaxf(fmaxf(s[par][0][b][0], s[par][0][b][1]), s[par][0][b][2]);
    mx = fmaxf(fmaxf(mx, s[par][0][b][3]), s[par][1][b][0]);
    mx = fmaxf(fmaxf(mx, s[par][1][b][1]), s[par][1][b][2]);
    mxl[b] = fmaxf(mx, s[par][1][b][3]);
    pin_f(mxl[b]);
  };
  // cold: the bias tiles for sub-step u1, which meets (or lies beyond) the diagonal of this wave's rows
  auto set_bias = [&](int u1) {
#pragma unroll
    for (int a = 0; a < 2; a++)
#pragma unroll
      for (int b = 0; b < 4; b++)
#pragma unroll
        for (int r = 0; r < 4; r++) mb[a][b][r] = (32 * u1 + 16 * a + r > dlt[b]) ? -INFINITY : 0.f;
    settle_valu();
  };
  // cold: rescale the accumulators of the query tiles flagged one phase ago (every PV MFMA with the old scale is in)
  auto apply_pending = [&]() {
    retire_mfmas();
    retire_mfmas();
#pragma unroll
    for (int b = 0; b < 4; b++) {
      if (pend_mask & (1u << b)) {
#pragma unroll
        for (int c = 0; c < 8; c++) {
          pin_a(oacc[c][b]);
#pragma unroll
          for (int r = 0; r < 4; r++) oacc[c][b][r] *= pend[b];
          pin_a(oacc[c][b]);
        }
        pend[b] = 1.f;
      }
    }
    settle_valu();
    pend_mask = 0;
  };
  // cold: raise the running maximum of the query tiles whose checked scores outgrew it
  auto raise = [&]() {
#pragma unroll
    for (int b = 0; b < 4; b++) {
      if (__builtin_amdgcn_ballot_w64(mxl[b] > thr[b]) != 0) {
        const float m_new = fmaxf(m_i[b], quad_max(mxl[b]) * qk_scale);
        const float alpha = fast_exp2(m_i[b] - m_new);
        l_i[b] *= alpha;
        pend[b] *= alpha;
        m_i[b] = m_new;
        thr[b] = (m_new + RESCALE_LOG2) * inv_scale;
        pend_mask |= 1u << b;
      }
    }
  };
  auto any_raise = [&]() {
    return __builtin_amdgcn_ballot_w64((mxl[0] > thr[0]) | (mxl[1] > thr[1]) | (mxl[2] > thr[2]) | (mxl[3] > thr[3])) != 0;
  };
  // ring slot addresses of K tile `kb` / of V tile `vb`
  auto set_kslot = [&](int kb) {
    const unsigned ko = (unsigned)((kb % KNS) * TILE);
#pragma unroll
    for (int ks = 0; ks < 4; ks++) kad[ks] = (ka ^ (ks << 6)) + ko;
  };
  auto set_vslot = [&](int vb) {
    const unsigned vo = (unsigned)((vb % VNS) * TILE);
#pragma unroll
    for (int c = 0; c < 8; c++) vad[c] = (va ^ (c << 5)) + vo;
  };

  using I0 = std::integral_constant<int, 0>;
  using I1 = std::integral_constant<int, 1>;
  using T = std::true_type;
  using F = std::false_type;

  // One phase.  PAR = u & 1: X(u) reads S buffer PAR and writes P buffer PAR; S(u+1) writes S buffer PAR ^ 1 from
  // the half PAR ^ 1 of its K tile; PV(u-1) reads P buffer PAR ^ 1 and the half PAR ^ 1 of its V tile.
  // Entry: the first two K fragments of S(u+1) have been requested (kf[0], kf[1]).  Exit: those of S(u+2).
  // Even phases hold the barrier X_j (j = u / 2) between their two parts, switch the K addresses to tile j + 1
  // behind it, and the loads of the group behind it (V tile j + 2, K tile j + 3) are issued one behind every
  // fourth MFMA of their PV part and of the next phase's S part.
  auto phase = [&](auto PAR_, auto DO_S_, auto DO_X_, auto DO_PV_, int u) {
    constexpr int par = decltype(PAR_)::value;
    constexpr bool do_s = decltype(DO_S_)::value, do_x = decltype(DO_X_)::value, do_pv = decltype(DO_PV_)::value;
    using HK = std::integral_constant<int, par ^ 1>;   // half of the K tile of S(u+1) and of the V tile of PV(u-1)
    using HN = std::integral_constant<int, par>;       // half of the K tile of S(u+2)
    const int j = u >> 1;
    // ---- S part: 32 MFMAs, fragment n = 2 ks + a feeds the four query tiles
    static_for<8>([&](auto N_) {
      constexpr int n = decltype(N_)::value, ks = n >> 1, a = n & 1;
      if constexpr (do_s) {
        if constexpr (n + 2 < 8) read_k(std::integral_constant<int, n + 2>{}, HK{}, kf[(n + 2) % 3]);
        else if constexpr (do_pv) read_v(std::integral_constant<int, n + 2 - 8>{}, HK{}, vf[(n + 2 - 8) % 3]);
        // reads issued behind fragment n: two K reads, or one K read and a V fragment (two reads), or two V fragments
        if constexpr (n + 2 < 8) lds_wait<2>();
        else if constexpr (!do_pv) lds_wait<7 - n>();
        else if constexpr (n == 6) lds_wait<3>();
        else lds_wait<4>();
        lds_use(kf[n % 3]);
      } else if constexpr (do_pv && n >= 6) {
        read_v(std::integral_constant<int, n - 6>{}, HK{}, vf[(n - 6) % 3]);
      }
      static_for<4>([&](auto B_) {
        constexpr int b = decltype(B_)::value, slot = n * 4 + b;
        if constexpr (do_s) {
          if constexpr (ks == 0) mfma16_s_first<BF>(s[par ^ 1][a][b], kf[n % 3], qf[b][ks], mb[a][b]);
          else mfma16_s_acc<BF>(s[par ^ 1][a][b], kf[n % 3], qf[b][ks]);
        }
        if constexpr (do_x && (slot & 1) == 0) x_elem(PAR_, std::integral_constant<int, slot / 2>{});
        if constexpr (par == 1 && (slot & 3) == 3 && slot / 4 >= 4) {
          // second half of the load group issued behind barrier X_j of the phase before: K tile j + 3
          if constexpr ((MI355_P16_KO & 8) == 0) load_k(std::integral_constant<int, slot / 4 - 4>{}, j + 3, F{});
        }
        __builtin_amdgcn_sched_barrier(0);
      });
    });
    if constexpr (par == 0) {
      // X_j: every wave is done with K tile j (and V tile j - 2), and has seen its share of K tile j + 1 and V tile j
      // arrive (the group behind X_{j-1} may still be in flight)
      wait_vmcnt<GROUP>();
      __builtin_amdgcn_sched_barrier(0);
      block_barrier();
      __builtin_amdgcn_sched_barrier(0);
      set_kslot(j + 1);
    }
    // ---- PV part: 32 MFMAs, fragment c feeds the four query tiles; the first two K fragments of the next phase's
    // S part are requested behind the last V fragments
    static_for<8>([&](auto C_) {
      constexpr int c = decltype(C_)::value;
      if constexpr (do_pv) {
        if constexpr (c + 2 < 8) read_v(std::integral_constant<int, c + 2>{}, HK{}, vf[(c + 2) % 3]);
        else read_k(std::integral_constant<int, c - 6>{}, HN{}, kf[c - 6]);
        if constexpr (c + 2 < 8) lds_wait<4>();
        else if constexpr (c == 6) lds_wait<3>();
        else lds_wait<2>();
        lds_use(vf[c % 3][0]);
        lds_use(vf[c % 3][1]);
      } else if constexpr (do_s && c >= 6) {
        read_k(std::integral_constant<int, c - 6>{}, HN{}, kf[c - 6]);
      }
      const i32x4 vfrag = __builtin_shufflevector(vf[c % 3][0], vf[c % 3][1], 0, 1, 2, 3);
      static_for<4>([&](auto B_) {
        constexpr int b = decltype(B_)::value, slot = 32 + c * 4 + b;
        if constexpr (do_pv) mfma16_o<BF>(oacc[c][b], vfrag, pf[par ^ 1][b]);
        if constexpr (do_x && (slot & 1) == 0) x_elem(PAR_, std::integral_constant<int, slot / 2>{});
        if constexpr (do_s && slot >= 44 && slot < 60 && (slot & 3) == 0) check_b(HK{}, std::integral_constant<int, (slot - 44) / 4>{});
        if constexpr (par == 0 && (slot & 3) == 3 && (slot - 32) / 4 < 4) {
          // first half of the load group behind X_j: V tile j + 2
          if constexpr ((MI355_P16_KO & 8) == 0) load_v(std::integral_constant<int, (slot - 32) / 4>{}, j + 2, F{});
        }
        __builtin_amdgcn_sched_barrier(0);
      });
    });
    if constexpr (par == 0) set_vslot(j);   // the V tile of PV(u), PV(u+1)
  };
  // the cold work between two phases: the accumulators' pending rescale, the raise that the scores of S(u+1) ask
  // for, and the bias tiles of S(u+2) where that sub-step meets the diagonal
  auto between = [&](int u, bool more_s) {
    if (pend_mask) apply_pending();
    if (more_s && any_raise()) raise();
    if (u + 2 >= first_masked) set_bias(u + 2);
  };

  // ---- prologue: V tiles 0, 1 and K tiles 0, 1, 2; S(0) alone; its check
#pragma unroll
  for (int blk = 0; blk < 2; blk++) static_for<INST>([&](auto I_) { load_v(I_, blk, T{}); });
#pragma unroll
  for (int blk = 0; blk < 3; blk++) static_for<INST>([&](auto I_) { load_k(I_, blk, T{}); });
  wait_vmcnt<0>();
  __builtin_amdgcn_sched_barrier(0);
  block_barrier();
  __builtin_amdgcn_sched_barrier(0);
  set_kslot(0);
  set_vslot(0);
  if (first_masked == 0) set_bias(0);
  {
    // S(0) into buffer 0 from the first half of K tile 0
    read_k(I0{}, I0{}, kf[0]);
    read_k(I1{}, I0{}, kf[1]);
    static_for<8>([&](auto N_) {
      constexpr int n = decltype(N_)::value, ks = n >> 1, a = n & 1;
      if constexpr (n + 2 < 8) read_k(std::integral_constant<int, n + 2>{}, I0{}, kf[(n + 2) % 3]);
      if constexpr (n + 2 < 8) lds_wait<2>();
      else lds_wait<7 - n>();
      lds_use(kf[n % 3]);
      static_for<4>([&](auto B_) {
        constexpr int b = decltype(B_)::value;
        if constexpr (ks == 0) mfma16_s_first<BF>(s[0][a][b], kf[n % 3], qf[b][ks], mb[a][b]);
        else mfma16_s_acc<BF>(s[0][a][b], kf[n % 3], qf[b][ks]);
      });
      __builtin_amdgcn_sched_barrier(0);
    });
    retire_mfmas();
#pragma unroll
    for (int a = 0; a < 2; a++)
#pragma unroll
      for (int b = 0; b < 4; b++) pin_v(s[0][a][b]);
    static_for<4>([&](auto B_) { check_b(I0{}, B_); });
    if (any_raise()) raise();
    if (1 >= first_masked) set_bias(1);
    // the first two K fragments of S(1)
    read_k(I0{}, I1{}, kf[0]);
    read_k(I1{}, I1{}, kf[1]);
  }

  // ---- the phases.  L is odd: phase 0 (no PV yet), then pairs of full phases (u odd, u + 1 even) while S(u + 2)
  // is still wanted, then this wave's two last phases L (X and PV) and L + 1 (PV), then - while other waves of the
  // workgroup still multiply - phases that only keep up this wave's share of the loads and of the barriers.
  const int nphases = 2 * nblocks + 1;
  phase(I0{}, T{}, T{}, F{}, 0);
  between(0, true);
  int u = 1;
  for (; u + 1 < L; u += 2) {
    phase(I1{}, T{}, T{}, T{}, u);
    between(u, true);
    phase(I0{}, T{}, T{}, T{}, u + 1);
    between(u + 1, true);
  }
  phase(I1{}, F{}, T{}, T{}, u);         // u == L
  between(u, false);
  phase(I0{}, F{}, F{}, T{}, u + 1);
  u += 2;
  for (; u < nphases; u += 2) {
    phase(I1{}, F{}, F{}, F{}, u);
    phase(I0{}, F{}, F{}, F{}, u + 1);
  }
  // nothing may still be writing this workgroup's LDS when it retires, and no fragment read may be in flight
  wait_all();
#pragma unroll
  for (int i = 0; i < 3; i++) { lds_use(kf[i]); lds_use(vf[i][0]); lds_use(vf[i][1]); }

  // ---- epilogue: O = acc / l, M = m + log2(l)
  retire_mfmas();
  retire_mfmas();
#pragma unroll
  for (int b = 0; b < 4; b++) {
    const float l = quad_sum(l_i[b]);
    const int row = row0 + b * 16 + l16;
    const float inv = pend[b] / l;        // (a rescale still pending is applied here)
    if (kg == 0) p.lse[(int64_t)hz * p.N + row] = m_i[b] + log2f(l);
    char* dst = obase + (int64_t)row * opitch + kg * 8;
    typedef __attribute__((ext_vector_type(4))) S S4;
#pragma unroll
    for (int c = 0; c < 8; c++) {
      pin_a(oacc[c][b]);
      S4 v;
#pragma unroll
      for (int e = 0; e < 4; e++) v[e] = (S)(oacc[c][b][e] * inv);
      *(S4*)(dst + c * 32) = v;
    }
  }
}

template <typename S, bool BF>
static int launch_fwd_p16(const AttnArgs& p, hipStream_t stream) {
  constexpr int BM = 256, smem = (3 + 4) * 64 * 256;
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)attn_fwd_p16_kernel<S, BF>, hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) return (int)e;
    attr_set = true;
  }
  const int nqb = p.N / BM;
  attn_fwd_p16_kernel<S, BF><<<dim3(nqb * p.Z * p.H), dim3(256), smem, stream>>>(p);
  return (int)hipGetLastError();
}

// head_dim 128, N_CTX a multiple of 256, a positive softmax scale
bool attn_fwd_p16_ok(const AttnArgs& p) {
  return p.D == 128 && p.d_real == 128 && p.N % 256 == 0 && p.sm_scale > 0.f;
}

int attn_fwd_p16_launch(const AttnArgs& p, bool bf16, hipStream_t stream) {
  return bf16 ? launch_fwd_p16<__bf16, true>(p, stream) : launch_fwd_p16<_Float16, false>(p, stream);
}

}  // namespace mi355

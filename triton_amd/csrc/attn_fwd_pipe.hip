// Fused flash-attention forward for gfx950, head_dim 128, software pipelined inside each wave.
//
// Same algorithm as the reference `_attn_fwd` / `_attn_fwd_inner` (python/tutorials/06-fused-attention.py:25-75,
// :98-187) and as attn_fwd.hip: online softmax in fp32 in the exp2 domain with qk_scale = sm_scale * 1.44269504
// (:160-161), P rounded to the input type before the second product (:66-70) while the normaliser sums the
// unrounded P (:57-58), causal blocks above the diagonal skipped and only the diagonal masked (:33-40, :49-53),
// M = m + log2(l), O = acc / l at the end (:183-187).  What differs is how the work is laid over the machine:
//
//   * a workgroup is four waves, ONE per SIMD, each owning 64 query rows (two 32-row tiles b) and all of head_dim,
//     so a K or V fragment read from LDS feeds two 32x32x16 MFMAs - half the LDS bytes per flop of a 32-row wave.
//     Scores are computed transposed (S^T = K Q^T), so a lane holds 16 scores of ONE query row per tile and the
//     16-bit P^T registers are, as they stand, the B operand of O^T += V^T P^T (attn_fwd.hip's layouts);
//   * what bounds such a kernel is instruction issue: measured on one wave, a 32x32x16 MFMA occupies the issue port
//     for 8 of its 32 cycles, a vector instruction for 4, an exponential for 8 - so a 32-cycle MFMA slot has room for
//     six vector instructions and the softmax of a score (multiply-add, exponential, sum, half a conversion: 18
//     cycles) fits one slot, while 16x16x32 MFMAs, cheaper in energy, leave only 8 of 16 cycles and do not;
//   * with one wave per SIMD nothing overlaps for free, so the key loop is a three-stage pipeline over sub-steps
//     u of 32 keys:  phase(u) = [ S(u+1): 16 MFMAs | PV(u-1): 16 MFMAs ] with the softmax arithmetic X(u) - itself
//     pipelined element by element, so that no instruction waits for the one before it - and every LDS read and
//     global load threaded between them.  S and P are double buffered in architectural registers; the O
//     accumulators and the Q fragments live in the accumulation registers, pinned there by issuing every MFMA as
//     inline assembly;
//   * the causal mask costs no instruction: the first MFMA of a score tile starts from a bias tile that is zero, or
//     -inf where a key is hidden, recomputed (cold) for the two sub-steps of a wave that meet the diagonal;
//   * the running maximum is lazy (raised only when a score outgrows it by more than 2^8), and the test for that is
//     per lane against a precomputed threshold - no cross-lane traffic on the hot path.  Raising it is a cold
//     branch between two phases: m and l change at once (X(u+1) uses them), the O accumulators are rescaled one
//     phase later, behind the PV MFMAs that still carry the old scale;
//   * K tiles (64 keys) go through a ring of three LDS stages, V tiles through a ring of four, filled by direct
//     global->LDS loads two to three tiles ahead; one workgroup barrier per 64 keys, placed between the S part and
//     the PV part of the even phases where every fragment read on either side of it is of a tile that landed long ago.
#include "attn_tiles.h"
#include "launch.h"

// Build-time knock-outs for timing experiments (results are wrong with any of them set): 1 = no softmax arithmetic,
// 2 = no maximum check, 4 = no LDS fragment reads, 8 = no global loads, 16 = no MFMAs.
#ifndef MI355_ATTN_PIPE_KO
#define MI355_ATTN_PIPE_KO 0
#endif
// Build-time switch for a timing experiment: the waves accumulate shader-clock cycles per part of the main loop's
// phases and workgroup 0 writes its sums over M (which is wrong then).
// 1: the main loop's phases with each pair of MFMA slots as one assembly statement; 0: as separate statements
#ifndef MI355_ATTN_PIPE_FUSED_SLOTS
#define MI355_ATTN_PIPE_FUSED_SLOTS 1
#endif
#ifndef MI355_ATTN_PIPE_TIMING
#define MI355_ATTN_PIPE_TIMING 0
#endif

namespace mi355 {

namespace {

// ---- MFMAs as inline assembly (operand register files are fixed by the constraints: v = architectural, a = accumulation)
// (the first k-step of a score tile starts from a bias tile: zeros, or -inf where the causal mask hides a key)
template <bool BF>
__device__ __forceinline__ void mfma32_s_first(f32x16& d, const i32x4& k, const i32x4& q, const f32x16& bias) {
#if MI355_DEVICE_PASS
  if constexpr ((MI355_ATTN_PIPE_KO & 16) != 0) { d = bias; return; }
  if constexpr (BF) asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %3" : "=&v"(d) : "v"(k), "a"(q), "v"(bias));
  else asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %3" : "=&v"(d) : "v"(k), "a"(q), "v"(bias));
#endif
}
template <bool BF>
__device__ __forceinline__ void mfma32_s_acc(f32x16& d, const i32x4& k, const i32x4& q) {
#if MI355_DEVICE_PASS
  if constexpr ((MI355_ATTN_PIPE_KO & 16) != 0) return;
  if constexpr (BF) asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(d) : "v"(k), "a"(q));
  else asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(d) : "v"(k), "a"(q));
#endif
}
template <bool BF>
__device__ __forceinline__ void mfma32_o(f32x16& d, const i32x4& v, const i32x4& pt) {
#if MI355_DEVICE_PASS
  if constexpr ((MI355_ATTN_PIPE_KO & 16) != 0) return;
  if constexpr (BF) asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(d) : "v"(v), "v"(pt));
  else asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(d) : "v"(v), "v"(pt));
#endif
}
// every MFMA issued so far has written its result once two of these have passed (2 x 16 idle slots)
__device__ __forceinline__ void retire_mfmas() {
#if MI355_DEVICE_PASS
  asm volatile("s_nop 15" ::: "memory");
#endif
}
__device__ __forceinline__ void pin_a(f32x16& x) {
#if MI355_DEVICE_PASS
  asm volatile("" : "+a"(x));
#endif
}
__device__ __forceinline__ void pin_v(f32x16& x) {
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

__device__ __forceinline__ unsigned long long stamp() {
  unsigned long long t = 0;
#if MI355_DEVICE_PASS && MI355_ATTN_PIPE_TIMING
  asm volatile("s_memtime %0" : "=s"(t));
#endif
  return t;
}

template <typename S>
__device__ __forceinline__ int pack2(float x, float y) {
  typedef __attribute__((ext_vector_type(2))) S S2;
  return __builtin_bit_cast(int, S2{(S)x, (S)y});
}


// ---- One pair of MFMA slots as ONE assembly statement (the full phases of the key loop): the wait for the pair's
// fragment, the two MFMAs on it (query tiles 0 and 1), and behind each its slice of the softmax pipeline - finish
// element i (sum, and with CVT the conversion of a pair of probabilities), exponentiate element i + 1, start element
// i + 2 - plus, in the PV part, one step of the maximum of the next sub-step's scores.  Written out because what
// bounds this kernel is instruction issue: measured on the device, a 32-cycle MFMA slot hides about 24 cycles of
// other instructions (4 per vector instruction, 8 per exponential) and every cycle beyond that is paid in full,
// and around statements of its own the compiler pads uses of assembly results with idle slots (79 per phase).
// sA .. sD: scores [tile 0, r], [tile 1, r], [tile 0, r + 1], [tile 1, r + 1] of the sub-step being exponentiated;
// sP0 / sP1: [tile 0 / 1, r - 1] (CVT: r odd).  Distances inside: an exponential is read two or more instructions
// later, a multiply-add result three or more.
#define MI355_X_SLOT0(CVS) "v_add_f32 %[l0], %[sA], %[l0]\n\t" CVS "v_exp_f32 %[sB], %[sB]\n\tv_fma_f32 %[sC], %[sC], %[sc], -%[m0]\n\t"
#define MI355_X_SLOT1(CVS) "v_add_f32 %[l1], %[sB], %[l1]\n\t" CVS "v_exp_f32 %[sC], %[sC]\n\tv_fma_f32 %[sD], %[sD], %[sc], -%[m1]\n\t"
#define MI355_WAITL "s_waitcnt lgkmcnt(%[n])\n\t"
#define MI355_X_OUT "+v"(l0), "+v"(l1), "+v"(sB), "+v"(sC), "+v"(sD)
#define MI355_X_IN [sA] "v"(sA), [sc] "s"(sc), [m0] "v"(m0), [m1] "v"(m1), [n] "i"(N)

// S part: scores of the next sub-step, tiles 0 and 1, k-step of fragment `fr`; FIRST: from the bias tiles
template <bool BF, bool FIRST, bool CVT, int N>
__device__ __forceinline__ void pair_s(f32x16& a0, f32x16& a1, const i32x4& fr, const i32x4& q0, const i32x4& q1, const f32x16& bi0,
                                       const f32x16& bi1, float& l0, float& l1, float sA, float& sB, float& sC, float& sD, float sP0, float sP1,
                                       int& w0, int& w1, float sc, float m0, float m1) {
#if MI355_DEVICE_PASS
#define MI355_PAIR_S(T, CV)                                                                                                        \
  if constexpr (FIRST)                                                                                                             \
    asm volatile(MI355_WAITL "v_mfma_f32_32x32x16_" T " %[a0], %[fr], %[q0], %[bi0]\n\t" MI355_X_SLOT0("")                        \
                 "v_mfma_f32_32x32x16_" T " %[a1], %[fr], %[q1], %[bi1]\n\t" MI355_X_SLOT1("")                                    \
                 : [a0] "=&v"(a0), [a1] "=&v"(a1), [l0] "+v"(l0), [l1] "+v"(l1), [sB] "+v"(sB), [sC] "+v"(sC), [sD] "+v"(sD)      \
                 : [fr] "v"(fr), [q0] "a"(q0), [q1] "a"(q1), [bi0] "v"(bi0), [bi1] "v"(bi1), MI355_X_IN);                         \
  else if constexpr (CVT)                                                                                                          \
    asm volatile(MI355_WAITL "v_mfma_f32_32x32x16_" T " %[a0], %[fr], %[q0], %[a0]\n\t" MI355_X_SLOT0(CV " %[w0], %[sP0], %[sA]\n\t") \
                 "v_mfma_f32_32x32x16_" T " %[a1], %[fr], %[q1], %[a1]\n\t" MI355_X_SLOT1(CV " %[w1], %[sP1], %[sB]\n\t")         \
                 : [a0] "+v"(a0), [a1] "+v"(a1), [l0] "+v"(l0), [l1] "+v"(l1), [sB] "+v"(sB), [sC] "+v"(sC), [sD] "+v"(sD),       \
                   [w0] "=&v"(w0), [w1] "=&v"(w1)                                                                                 \
                 : [fr] "v"(fr), [q0] "a"(q0), [q1] "a"(q1), [sP0] "v"(sP0), [sP1] "v"(sP1), MI355_X_IN);                         \
  else                                                                                                                             \
    asm volatile(MI355_WAITL "v_mfma_f32_32x32x16_" T " %[a0], %[fr], %[q0], %[a0]\n\t" MI355_X_SLOT0("")                         \
                 "v_mfma_f32_32x32x16_" T " %[a1], %[fr], %[q1], %[a1]\n\t" MI355_X_SLOT1("")                                     \
                 : [a0] "+v"(a0), [a1] "+v"(a1), [l0] "+v"(l0), [l1] "+v"(l1), [sB] "+v"(sB), [sC] "+v"(sC), [sD] "+v"(sD)        \
                 : [fr] "v"(fr), [q0] "a"(q0), [q1] "a"(q1), MI355_X_IN)
  if constexpr (BF) { MI355_PAIR_S("bf16", "v_cvt_pk_bf16_f32"); } else { MI355_PAIR_S("f16", "v_cvt_pk_f16_f32"); }
#undef MI355_PAIR_S
#endif
}

// PV part: O^T tiles 0 and 1 += V^T fragment `fr` times P^T operands p0 / p1, and step CHK of the lane's maximum of
// the next sub-step's scores (ca*: two registers of its tile 0, cb*: of its tile 1; CHK == 1: the first step)
template <bool BF, bool CVT, int CHK, int N>
__device__ __forceinline__ void pair_pv(f32x16& a0, f32x16& a1, const i32x4& fr, const i32x4& p0, const i32x4& p1, float& l0, float& l1,
                                        float sA, float& sB, float& sC, float& sD, float sP0, float sP1, int& w0, int& w1, float sc,
                                        float m0, float m1, float& mx0, float& mx1, float ca0, float ca1, float cb0, float cb1) {
#if MI355_DEVICE_PASS
#define MI355_CHK0 "v_max3_f32 %[mx0], %[mx0], %[ca0], %[ca1]\n\t"
#define MI355_CHK1 "v_max3_f32 %[mx1], %[mx1], %[cb0], %[cb1]\n\t"
#define MI355_CHF0 "v_max_f32 %[mx0], %[ca0], %[ca1]\n\t"
#define MI355_CHF1 "v_max_f32 %[mx1], %[cb0], %[cb1]\n\t"
#define MI355_PAIR_PV(T, CV, K0, K1, MXC)                                                                                          \
  if constexpr (CVT)                                                                                                               \
    asm volatile(MI355_WAITL "v_mfma_f32_32x32x16_" T " %[a0], %[fr], %[p0], %[a0]\n\t" MI355_X_SLOT0(CV " %[w0], %[sP0], %[sA]\n\t") K0 \
                 "v_mfma_f32_32x32x16_" T " %[a1], %[fr], %[p1], %[a1]\n\t" MI355_X_SLOT1(CV " %[w1], %[sP1], %[sB]\n\t") K1      \
                 : [a0] "+a"(a0), [a1] "+a"(a1), [l0] "+v"(l0), [l1] "+v"(l1), [sB] "+v"(sB), [sC] "+v"(sC), [sD] "+v"(sD),       \
                   [w0] "=&v"(w0), [w1] "=&v"(w1), [mx0] MXC(mx0), [mx1] MXC(mx1)                                                 \
                 : [fr] "v"(fr), [p0] "v"(p0), [p1] "v"(p1), [sP0] "v"(sP0), [sP1] "v"(sP1), [ca0] "v"(ca0), [ca1] "v"(ca1),      \
                   [cb0] "v"(cb0), [cb1] "v"(cb1), MI355_X_IN);                                                                   \
  else                                                                                                                             \
    asm volatile(MI355_WAITL "v_mfma_f32_32x32x16_" T " %[a0], %[fr], %[p0], %[a0]\n\t" MI355_X_SLOT0("") K0                      \
                 "v_mfma_f32_32x32x16_" T " %[a1], %[fr], %[p1], %[a1]\n\t" MI355_X_SLOT1("") K1                                  \
                 : [a0] "+a"(a0), [a1] "+a"(a1), [l0] "+v"(l0), [l1] "+v"(l1), [sB] "+v"(sB), [sC] "+v"(sC), [sD] "+v"(sD),       \
                   [mx0] MXC(mx0), [mx1] MXC(mx1)                                                                                 \
                 : [fr] "v"(fr), [p0] "v"(p0), [p1] "v"(p1), [ca0] "v"(ca0), [ca1] "v"(ca1), [cb0] "v"(cb0), [cb1] "v"(cb1),      \
                   MI355_X_IN)
#define MI355_RW "+v"
#define MI355_WO "=&v"
  if constexpr (BF) {
    if constexpr (CHK == 1) { MI355_PAIR_PV("bf16", "v_cvt_pk_bf16_f32", MI355_CHF0, MI355_CHF1, MI355_WO); }
    else { MI355_PAIR_PV("bf16", "v_cvt_pk_bf16_f32", MI355_CHK0, MI355_CHK1, MI355_RW); }
  } else {
    if constexpr (CHK == 1) { MI355_PAIR_PV("f16", "v_cvt_pk_f16_f32", MI355_CHF0, MI355_CHF1, MI355_WO); }
    else { MI355_PAIR_PV("f16", "v_cvt_pk_f16_f32", MI355_CHK0, MI355_CHK1, MI355_RW); }
  }
#undef MI355_PAIR_PV
#endif
}

}  // namespace

template <typename S, bool BF>
__global__ __launch_bounds__(256, 1) void attn_fwd_pipe_kernel(AttnArgs p) {
  constexpr int NW = 4, BM = 256, BN = 64, RB = 256;
  using Tile = AttnTile<RB, BN, NW>;
  constexpr int TILE = Tile::BYTES;      // 16 KiB per K or V tile
  constexpr int KNS = 3, VNS = 4;        // ring depths
  constexpr int VBASE = KNS * TILE;
  constexpr int INST = Tile::INST;       // direct loads per wave and tile (4)
  constexpr int GROUP = 2 * INST;        // loads per wave and 64 keys
  constexpr float RESCALE_LOG2 = 8.f;

  extern __shared__ __attribute__((aligned(1024))) char smem[];
  const unsigned lds0 = lds_addr((LDS_PTR(const void))smem);

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, g = lane >> 5, i16 = lane & 15, q4 = lane >> 4;

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
  const int L = p.causal ? (row0 + 63) / 32 : 2 * nblocks - 1;     // this wave's last sub-step (odd)
  const int first_masked = p.causal ? row0 / 32 : 2 * nblocks;     // its first sub-step that meets the diagonal

  // ---- Q fragments (B operand of S^T): lane (query l32 of tile b, half g) holds Q[row][16 ks + 8 g .. + 8]
  i32x4 qf[2][8];
#pragma unroll
  for (int b = 0; b < 2; b++) {
    const char* src = qbase + (int64_t)(row0 + b * 32 + l32) * qpitch + g * 16;
#pragma unroll
    for (int ks = 0; ks < 8; ks++) qf[b][ks] = *(const i32x4*)(src + ks * 32);
  }

  // ---- direct loads: a scalar tile base plus a 32-bit per-lane offset (attn_tiles.h)
  unsigned offK[INST], offV[INST];
#pragma unroll
  for (int i = 0; i < INST; i++) {
    offK[i] = (unsigned)Tile::off(kpitch, wave, lane, i);
    offV[i] = (unsigned)Tile::off(vpitch, wave, lane, i);
  }
  // source and destination of the loads of one tile are set once per tile (scalars): tile `blk` (clamped to the
  // workgroup's last) into its ring slot, this wave's share of each instruction at + wave KiB
  const int64_t kstep = (int64_t)BN * kpitch, vstep = (int64_t)BN * vpitch;
  const char* ksrc = kbase;
  const char* vsrc = vbase;
  unsigned kdst = lds0 + wave * 1024, vdst = lds0 + VBASE + wave * 1024;
  auto aim_k = [&](int blk) { ksrc = kbase + min(blk, nblocks - 1) * kstep; kdst = lds0 + (blk % KNS) * TILE + wave * 1024; };
  auto aim_v = [&](int blk) { vsrc = vbase + min(blk, nblocks - 1) * vstep; vdst = lds0 + VBASE + (blk % VNS) * TILE + wave * 1024; };
  auto load_k = [&](auto I_, auto SETTLE_) {
    constexpr int i = decltype(I_)::value;
    async_copy16_sbase<decltype(SETTLE_)::value>(ksrc, offK[i], kdst + i * NW * 1024);
  };
  auto load_v = [&](auto I_, auto SETTLE_) {
    constexpr int i = decltype(I_)::value;
    async_copy16_sbase<decltype(SETTLE_)::value>(vsrc, offV[i], vdst + i * NW * 1024);
  };

  // ---- fragment addresses (row-wise K operand per k-step, transposed V operand per column block and half); the
  // ring slot offsets are added per 64 keys, sub-step and k-step offsets ride in the instructions' immediates
  const RowRead<RB> rk(l32, g);
  const TrRead<RB> tv(i16, q4);
  unsigned kad[8], vad[4][2];        // addresses in the ring slots currently read

  // ---- state
  f32x16 oacc[4][2];                 // O^T tiles [d tile c][query tile b], accumulation registers
#pragma unroll
  for (int c = 0; c < 4; c++)
#pragma unroll
    for (int b = 0; b < 2; b++)
#pragma unroll
      for (int r = 0; r < 16; r++) oacc[c][b][r] = 0.f;
  f32x16 s[2][2];                    // S^T [buffer][query tile b]: 32 keys x 32 queries
  i32x4 pf[2][2][2];                 // P^T [buffer][query tile b][16-key k-step t]: B operand of the second product
#pragma unroll
  for (int b = 0; b < 2; b++)
#pragma unroll
    for (int t = 0; t < 2; t++) pf[1][b][t] = i32x4{0, 0, 0, 0};
  constexpr int FD = 4, NF = FD + 1; // fragments requested ahead of their MFMAs, and the registers for them
  i32x4 kf[NF];                      // K fragments in flight
  i32x2 vf[NF][2];                   // V^T fragments in flight (two transpose reads each)
  float m_i[2], l_i[2], thr[2], pend[2], mxl[2];
  unsigned long long over[2] = {0, 0};   // lanes whose checked scores outgrow the running maximum, per query tile
#pragma unroll
  for (int b = 0; b < 2; b++) { m_i[b] = -INFINITY; l_i[b] = 0.f; thr[b] = -INFINITY; pend[b] = 1.f; mxl[b] = -INFINITY; }
  unsigned pend_mask = 0;            // query tiles whose O accumulators await a rescale (wave-uniform)
  const float qk_scale = p.sm_scale * 1.44269504f;
  const float inv_scale = 1.f / qk_scale;
  // causal: register r of a score tile is key 32 u + 8 (r >> 2) + 4 g + (r & 3); it is hidden from this lane's query
  // row when 32 u + 8 (r >> 2) + (r & 3) exceeds dlt[b]
  int dlt[2];
#pragma unroll
  for (int b = 0; b < 2; b++) dlt[b] = row0 + 32 * b + l32 - 4 * g;
  f32x16 mb[2];                      // bias tiles of the scores per query tile b: 0, or -inf where masked
#pragma unroll
  for (int b = 0; b < 2; b++)
#pragma unroll
    for (int r = 0; r < 16; r++) mb[b][r] = 0.f;

  // ---- pieces of a phase
  // fragment reads: K fragment ks of the half HK of the current K slot; V fragment n = 4 t + c of the half HV
  auto read_k = [&](auto KS_, auto HK_, i32x4& dst) {
    constexpr int ks = decltype(KS_)::value, hk = decltype(HK_)::value;
    if constexpr ((MI355_ATTN_PIPE_KO & 4) == 0) dst = lds_read_b128<hk * 32 * RB>(kad[ks]);
  };
  auto read_v = [&](auto N_, auto HV_, i32x2 (&dst)[2]) {
    constexpr int n = decltype(N_)::value, t = n >> 2, c = n & 3, hv = decltype(HV_)::value;
    if constexpr ((MI355_ATTN_PIPE_KO & 4) != 0) return;
    dst[0] = lds_read_tr16_b64<(hv * 32 + 16 * t) * RB>(vad[c][0]);
    dst[1] = lds_read_tr16_b64<(hv * 32 + 16 * t + 8) * RB>(vad[c][1]);
  };
  // X, pipelined element by element: element e = 0 .. 31 of the sub-step whose scores sit in buffer PAR is register
  // r = e >> 1 of query tile b = e & 1.  x_fma(e), x_exp(e), x_fin(e) are issued in three consecutive MFMA slots, so
  // that no instruction of a slot waits for the one in front of it; consecutive elements alternate between the
  // tiles, so neither do the additions into l_i[b].
  auto x_fma = [&](auto PAR_, auto E_) {
    constexpr int par = decltype(PAR_)::value, e = decltype(E_)::value, b = e & 1, r = e >> 1;
    if constexpr ((MI355_ATTN_PIPE_KO & 1) != 0 || e < 0 || e > 31) return;
    else {
      pin_v(s[par][b]);
      s[par][b][r] = fmaf(s[par][b][r], qk_scale, -m_i[b]);
    }
  };
  auto x_exp = [&](auto PAR_, auto E_) {
    constexpr int par = decltype(PAR_)::value, e = decltype(E_)::value, b = e & 1, r = e >> 1;
    if constexpr ((MI355_ATTN_PIPE_KO & 1) != 0 || e < 0 || e > 31) return;
    else {
      pin_v(s[par][b]);
      s[par][b][r] = fast_exp2(s[par][b][r]);
    }
  };
  auto x_fin = [&](auto PAR_, auto E_) {
    constexpr int par = decltype(PAR_)::value, e = decltype(E_)::value, b = e & 1, r = e >> 1;
    if constexpr ((MI355_ATTN_PIPE_KO & 1) != 0 || e < 0 || e > 31) return;
    else {
      pin_v(s[par][b]);
      l_i[b] += s[par][b][r];
      pin_f(l_i[b]);
      if constexpr ((r & 1) == 1) {
        // k-step t = r >> 3 of the second product takes registers 8 t .. 8 t + 7 of the tile
        int w = pack2<S>(s[par][b][r - 1], s[par][b][r]);
        pin_i(w);
        pf[par][b][r >> 3][(r & 7) >> 1] = w;
      }
    }
  };
  // slot i of a phase: finish element i, exponentiate element i + 1, start element i + 2 (x_head, in front of the
  // phase's first MFMA, starts elements 0 and 1 and exponentiates element 0: the last slot leaves nothing behind)
  auto x_slot = [&](auto PAR_, auto I_) {
    constexpr int i = decltype(I_)::value;
    x_fin(PAR_, std::integral_constant<int, i>{});
    x_exp(PAR_, std::integral_constant<int, i + 1>{});
    x_fma(PAR_, std::integral_constant<int, i + 2>{});
  };
  auto x_head = [&](auto PAR_) {
    x_fma(PAR_, std::integral_constant<int, 0>{});
    x_fma(PAR_, std::integral_constant<int, 1>{});
    x_exp(PAR_, std::integral_constant<int, 0>{});
  };
  // the lane's largest score of query tile b in buffer PAR, in eight steps I = 0 .. 7 of two registers each
  auto check_step = [&](auto PAR_, auto B_, auto I_) {
    constexpr int par = decltype(PAR_)::value, b = decltype(B_)::value, i = decltype(I_)::value;
    if constexpr ((MI355_ATTN_PIPE_KO & 2) != 0) return;
    pin_v(s[par][b]);
    if constexpr (i == 0) mxl[b] = fmaxf(s[par][b][0], s[par][b][1]);
    else mxl[b] = fmaxf(fmaxf(mxl[b], s[par][b][2 * i]), s[par][b][2 * i + 1]);
    pin_f(mxl[b]);
    if constexpr (i == 7) over[b] = __builtin_amdgcn_ballot_w64(mxl[b] > thr[b]);
  };
  // cold: the bias tiles for sub-step u1, which meets (or lies beyond) the diagonal of this wave's rows
  auto set_bias = [&](int u1) {
#pragma unroll
    for (int b = 0; b < 2; b++)
#pragma unroll
      for (int r = 0; r < 16; r++) mb[b][r] = (32 * u1 + 8 * (r >> 2) + (r & 3) > dlt[b]) ? -INFINITY : 0.f;
    settle_valu();
  };
  // cold: rescale the accumulators of the query tiles flagged one phase ago (every PV MFMA with the old scale is in)
  auto apply_pending = [&]() {
    retire_mfmas();
    retire_mfmas();
#pragma unroll
    for (int b = 0; b < 2; b++) {
      if (pend_mask & (1u << b)) {
#pragma unroll
        for (int c = 0; c < 4; c++) {
          pin_a(oacc[c][b]);
#pragma unroll
          for (int r = 0; r < 16; r++) oacc[c][b][r] *= pend[b];
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
    for (int b = 0; b < 2; b++) {
      if (over[b] != 0) {
        const float m_new = fmaxf(m_i[b], pair_max(mxl[b]) * qk_scale);
        const float alpha = fast_exp2(m_i[b] - m_new);
        l_i[b] *= alpha;
        pend[b] *= alpha;
        m_i[b] = m_new;
        thr[b] = (m_new + RESCALE_LOG2) * inv_scale;
        pend_mask |= 1u << b;
      }
    }
  };
  auto any_raise = [&]() { return (over[0] | over[1]) != 0; };
  // ring slot addresses of K tile `kb` / of V tile `vb`
  auto set_kslot = [&](int kb) {
    const unsigned ko = lds0 + (unsigned)((kb % KNS) * TILE);
#pragma unroll
    for (int ks = 0; ks < 8; ks++) kad[ks] = ko + rk.rowb + (rk.xk ^ (ks * 32));
  };
  auto set_vslot = [&](int vb) {
    const unsigned vo = lds0 + VBASE + (unsigned)((vb % VNS) * TILE);
#pragma unroll
    for (int c = 0; c < 4; c++)
#pragma unroll
      for (int h2 = 0; h2 < 2; h2++) vad[c][h2] = vo + (tv.tl ^ ((c << 6) | (h2 << 5)));
  };

  unsigned long long tsum[5] = {0, 0, 0, 0, 0}, tlast = 0;   // (timing experiment) cycles in S part, barrier, PV part, between; phases
  using I0 = std::integral_constant<int, 0>;
  using I1 = std::integral_constant<int, 1>;
  using T = std::true_type;
  using F = std::false_type;

  // One phase.  PAR = u & 1: X(u) reads S buffer PAR and writes P buffer PAR; S(u+1) writes S buffer PAR ^ 1 from
  // the half PAR ^ 1 of its K tile; PV(u-1) reads P buffer PAR ^ 1 and the half PAR ^ 1 of its V tile.
  // The fragments of a phase form one sequence q = 0 .. 15 (eight of K, eight of V; fragment q feeds the MFMAs of
  // slots 2 q and 2 q + 1) that runs on into the next phase's K fragments: fragment q + FD is requested in front of
  // slot 2 q, so a read has FD MFMA pairs to land.  Entry: K fragments 0 .. FD - 1 of S(u+1) have been requested.
  // Every phase that reads at all issues every read (a product that a phase does not compute leaves its fragments
  // unused), so the number of reads in flight behind a fragment is the same everywhere.
  // Even phases hold the barrier X_j (j = u / 2) between their two parts, switch the K addresses to tile j + 1
  // behind it, and the loads of the group behind it (V tile j + 2, K tile j + 3) are issued one behind every
  // other MFMA pair of their PV part and of the next phase's S part.
  auto phase = [&](auto PAR_, auto DO_S_, auto DO_X_, auto DO_PV_, int u) {
    constexpr int par = decltype(PAR_)::value;
    constexpr bool do_s = decltype(DO_S_)::value, do_x = decltype(DO_X_)::value, do_pv = decltype(DO_PV_)::value;
    constexpr bool reads = do_s || do_x || do_pv;
    using HK = std::integral_constant<int, par ^ 1>;   // half of the K tile of S(u+1) and of the V tile of PV(u-1)
    using HN = std::integral_constant<int, par>;       // half of the K tile of S(u+2)
    const int j = u >> 1;
    const unsigned long long a0 = stamp();
    // request fragment Q of the sequence (16 .. 19: the next phase's first K fragments)
    auto request = [&](auto Q_) {
      constexpr int q = decltype(Q_)::value;
      if constexpr (q < 8) read_k(std::integral_constant<int, q>{}, HK{}, kf[q % NF]);
      else if constexpr (q < 16) read_v(std::integral_constant<int, q - 8>{}, HK{}, vf[(q - 8) % NF]);
      else read_k(std::integral_constant<int, q - 16>{}, HN{}, kf[(q - 16) % NF]);
    };
    // LDS reads issued behind fragment q once fragment q + FD has been requested
    auto behind = [](int q) { int n = 0; for (int i = q + 1; i <= q + FD; i++) n += (i >= 8 && i < 16) ? 2 : 1; return n; };
    if constexpr (par == 1) aim_k(j + 3);
    if constexpr (do_x) x_head(PAR_);
    // ---- S part: 16 MFMAs, K fragment n feeds the two query tiles
    static_for<8>([&](auto N_) {
      constexpr int n = decltype(N_)::value;
      if constexpr (reads) {
        request(std::integral_constant<int, n + FD>{});
        lds_wait<behind(n)>();
        lds_use(kf[n % NF]);
      }
      static_for<2>([&](auto B_) {
        constexpr int b = decltype(B_)::value, slot = n * 2 + b;
        if constexpr (do_s) {
          if constexpr (n == 0) mfma32_s_first<BF>(s[par ^ 1][b], kf[n % NF], qf[b][n], mb[b]);
          else mfma32_s_acc<BF>(s[par ^ 1][b], kf[n % NF], qf[b][n]);
        }
        if constexpr (do_x) x_slot(PAR_, std::integral_constant<int, slot>{});
        if constexpr (par == 1 && b == 1 && n >= 4) {
          // second half of the load group issued behind barrier X_j of the phase before: K tile j + 3
          if constexpr ((MI355_ATTN_PIPE_KO & 8) == 0) load_k(std::integral_constant<int, (n >= 4 ? n - 4 : 0)>{}, F{});
        }
        __builtin_amdgcn_sched_barrier(0);
      });
    });
    const unsigned long long a1 = stamp();
    if constexpr (par == 0) {
      // X_j: every wave is done with K tile j (and V tile j - 2), and has seen its share of K tile j + 1 and V tile j
      // arrive (the group behind X_{j-1} may still be in flight)
      wait_vmcnt<GROUP>();
      __builtin_amdgcn_sched_barrier(0);
      block_barrier();
      __builtin_amdgcn_sched_barrier(0);
      set_kslot(j + 1);
      aim_v(j + 2);
    }
    const unsigned long long a2 = stamp();
    // ---- PV part: 16 MFMAs, V fragment n = 4 t + c feeds the two query tiles
    static_for<8>([&](auto N_) {
      constexpr int n = decltype(N_)::value, t = n >> 2, c = n & 3;
      if constexpr (reads) {
        request(std::integral_constant<int, 8 + n + FD>{});
        lds_wait<behind(8 + n)>();
        lds_use(vf[n % NF][0]);
        lds_use(vf[n % NF][1]);
      }
      const i32x4 vfrag = __builtin_shufflevector(vf[n % NF][0], vf[n % NF][1], 0, 1, 2, 3);
      static_for<2>([&](auto B_) {
        constexpr int b = decltype(B_)::value, slot = 16 + n * 2 + b;
        if constexpr (do_pv) mfma32_o<BF>(oacc[c][b], vfrag, pf[par ^ 1][b][t]);
        if constexpr (do_x) x_slot(PAR_, std::integral_constant<int, slot>{});
        // the maximum of S(u+1), whose last MFMAs were slots 14 (tile 0) and 15 (tile 1): one step per slot, tile 0 in
        // the odd slots from 17 on, tile 1 in the even slots from 18 on (its last step shares slot 31)
        if constexpr (do_s && slot >= 17 && (slot & 1) == 1) check_step(HK{}, I0{}, std::integral_constant<int, (slot >= 17 ? (slot - 17) / 2 : 0)>{});
        if constexpr (do_s && slot >= 18 && (slot & 1) == 0) check_step(HK{}, I1{}, std::integral_constant<int, (slot >= 18 ? (slot - 18) / 2 : 0)>{});
        if constexpr (do_s && slot == 31) check_step(HK{}, I1{}, std::integral_constant<int, 7>{});
        if constexpr (par == 0 && b == 1 && n < 4) {
          // first half of the load group behind X_j: V tile j + 2
          if constexpr ((MI355_ATTN_PIPE_KO & 8) == 0) load_v(std::integral_constant<int, (n < 4 ? n : 0)>{}, F{});
        }
        __builtin_amdgcn_sched_barrier(0);
      });
    });
    if constexpr (par == 0) set_vslot(j);   // the V tile of PV(u), PV(u+1)
    if constexpr (MI355_ATTN_PIPE_TIMING != 0) {
      unsigned long long a3 = stamp(), b0 = a0, b1 = a1, b2 = a2;
      asm volatile("s_waitcnt lgkmcnt(0)" : "+s"(b0), "+s"(b1), "+s"(b2), "+s"(a3) :: "memory");
      tsum[0] += b1 - b0; tsum[1] += b2 - b1; tsum[2] += a3 - b2; tsum[4] += 1;
      tlast = a3;
    }
  };
  // The full phase (S, X and PV all present: every phase of the main loop) with each pair of MFMA slots as one
  // assembly statement (pair_s / pair_pv): same schedule as `phase`, same fragment sequence and loads.
  auto phase_full = [&](auto PAR_, int u) {
    constexpr int par = decltype(PAR_)::value;
    using HK = std::integral_constant<int, par ^ 1>;
    using HN = std::integral_constant<int, par>;
    const int j = u >> 1;
    auto request = [&](auto Q_) {
      constexpr int q = decltype(Q_)::value;
      if constexpr (q < 8) read_k(std::integral_constant<int, q>{}, HK{}, kf[q % NF]);
      else if constexpr (q < 16) read_v(std::integral_constant<int, q - 8>{}, HK{}, vf[(q - 8) % NF]);
      else read_k(std::integral_constant<int, q - 16>{}, HN{}, kf[(q - 16) % NF]);
    };
    auto behind = [](int q) { int n = 0; for (int i = q + 1; i <= q + FD; i++) n += (i >= 8 && i < 16) ? 2 : 1; return n; };
    if constexpr (par == 1) aim_k(j + 3);
    const unsigned long long a0 = stamp();
    x_head(PAR_);
    float dummy0 = 0.f, dummy1 = 0.f;
    // pair g = 0 .. 15: slots 2 g and 2 g + 1; elements [tile 0, g], [tile 1, g] are finished, [tile 0, g + 1], [tile 1, g + 1] started
    auto run_pair = [&](auto G_) {
      constexpr int g = decltype(G_)::value, n = g & 7;
      constexpr bool cvt = (g & 1) == 1;
      float sA = s[par][0][g], sB = s[par][1][g];
      float sC = g < 15 ? s[par][0][g < 15 ? g + 1 : 0] : dummy0, sD = g < 15 ? s[par][1][g < 15 ? g + 1 : 0] : dummy1;
      const float sP0 = s[par][0][g > 0 ? g - 1 : 0], sP1 = s[par][1][g > 0 ? g - 1 : 0];
      int w0 = 0, w1 = 0;
      request(std::integral_constant<int, g + FD>{});
      if constexpr (g < 8) {
        pair_s<BF, g == 0, cvt, behind(g)>(s[par ^ 1][0], s[par ^ 1][1], kf[n % NF], qf[0][n], qf[1][n], mb[0], mb[1], l_i[0], l_i[1],
                                           sA, sB, sC, sD, sP0, sP1, w0, w1, qk_scale, m_i[0], m_i[1]);
      } else {
        constexpr int t = n >> 2, c = n & 3, k = g - 8;
        const i32x4 vfrag = __builtin_shufflevector(vf[n % NF][0], vf[n % NF][1], 0, 1, 2, 3);
        pair_pv<BF, cvt, (k == 0 ? 1 : 2), behind(g)>(oacc[c][0], oacc[c][1], vfrag, pf[par ^ 1][0][t], pf[par ^ 1][1][t], l_i[0], l_i[1],
                                                      sA, sB, sC, sD, sP0, sP1, w0, w1, qk_scale, m_i[0], m_i[1], mxl[0], mxl[1],
                                                      s[par ^ 1][0][2 * k], s[par ^ 1][0][2 * k + 1], s[par ^ 1][1][2 * k], s[par ^ 1][1][2 * k + 1]);
      }
      s[par][1][g] = sB;
      if constexpr (g < 15) { s[par][0][g + 1] = sC; s[par][1][g + 1] = sD; }
      else { dummy0 = sC; dummy1 = sD; }
      if constexpr (cvt) { pf[par][0][g >> 3][(g & 7) >> 1] = w0; pf[par][1][g >> 3][(g & 7) >> 1] = w1; }
      if constexpr (par == 1 && g >= 4 && g < 8) {
        if constexpr ((MI355_ATTN_PIPE_KO & 8) == 0) load_k(std::integral_constant<int, (g >= 4 && g < 8 ? g - 4 : 0)>{}, F{});
      }
      if constexpr (par == 0 && g >= 8 && g < 12) {
        if constexpr ((MI355_ATTN_PIPE_KO & 8) == 0) load_v(std::integral_constant<int, (g >= 8 && g < 12 ? g - 8 : 0)>{}, F{});
      }
      __builtin_amdgcn_sched_barrier(0);
    };
    static_for<8>([&](auto N_) { run_pair(N_); });
    const unsigned long long a1 = stamp();
    if constexpr (par == 0) {
      wait_vmcnt<GROUP>();
      __builtin_amdgcn_sched_barrier(0);
      block_barrier();
      __builtin_amdgcn_sched_barrier(0);
      set_kslot(j + 1);
      aim_v(j + 2);
    }
    const unsigned long long a2 = stamp();
    static_for<8>([&](auto N_) { run_pair(std::integral_constant<int, 8 + decltype(N_)::value>{}); });
    over[0] = __builtin_amdgcn_ballot_w64(mxl[0] > thr[0]);
    over[1] = __builtin_amdgcn_ballot_w64(mxl[1] > thr[1]);
    if constexpr (par == 0) set_vslot(j);
    if constexpr (MI355_ATTN_PIPE_TIMING != 0) {
      unsigned long long a3 = stamp(), b0 = a0, b1 = a1, b2 = a2;
      asm volatile("s_waitcnt lgkmcnt(0)" : "+s"(b0), "+s"(b1), "+s"(b2), "+s"(a3) :: "memory");
      tsum[0] += b1 - b0; tsum[1] += b2 - b1; tsum[2] += a3 - b2; tsum[4] += 1;
      tlast = a3;
    }
  };
  // the cold work between two phases: the accumulators' pending rescale, the raise that the scores of S(u+1) ask
  // for, and the bias tiles of S(u+2) where that sub-step meets the diagonal
  auto between = [&](int u, bool more_s) {
    if (pend_mask) apply_pending();
    if (more_s && any_raise()) raise();
    if (u + 2 >= first_masked) set_bias(u + 2);
    if constexpr (MI355_ATTN_PIPE_TIMING != 0) {
      unsigned long long a4 = stamp();
      asm volatile("s_waitcnt lgkmcnt(0)" : "+s"(a4) :: "memory");
      tsum[3] += a4 - tlast;
    }
  };

  // ---- prologue: V tiles 0, 1 and K tiles 0, 1, 2; S(0) alone; its check
#pragma unroll
  for (int blk = 0; blk < 2; blk++) { aim_v(blk); static_for<INST>([&](auto I_) { load_v(I_, T{}); }); }
#pragma unroll
  for (int blk = 0; blk < 3; blk++) { aim_k(blk); static_for<INST>([&](auto I_) { load_k(I_, T{}); }); }
  wait_vmcnt<0>();
  __builtin_amdgcn_sched_barrier(0);
  block_barrier();
  __builtin_amdgcn_sched_barrier(0);
  set_kslot(0);
  set_vslot(0);
  if (first_masked == 0) set_bias(0);
  {
    // S(0) into buffer 0 from the first half of K tile 0
    static_for<FD>([&](auto Q_) { read_k(Q_, I0{}, kf[decltype(Q_)::value % NF]); });
    static_for<8>([&](auto N_) {
      constexpr int n = decltype(N_)::value;
      if constexpr (n + FD < 8) read_k(std::integral_constant<int, (n + FD < 8 ? n + FD : 0)>{}, I0{}, kf[(n + FD) % NF]);
      if constexpr (n + FD < 8) lds_wait<FD>();
      else lds_wait<7 - n>();
      lds_use(kf[n % NF]);
      static_for<2>([&](auto B_) {
        constexpr int b = decltype(B_)::value;
        if constexpr (n == 0) mfma32_s_first<BF>(s[0][b], kf[n % NF], qf[b][n], mb[b]);
        else mfma32_s_acc<BF>(s[0][b], kf[n % NF], qf[b][n]);
      });
      __builtin_amdgcn_sched_barrier(0);
    });
    retire_mfmas();
    retire_mfmas();
    pin_v(s[0][0]);
    pin_v(s[0][1]);
    static_for<8>([&](auto I_) { check_step(I0{}, I0{}, I_); check_step(I0{}, I1{}, I_); });
    if (any_raise()) raise();
    if (1 >= first_masked) set_bias(1);
    // the first K fragments of S(1)
    static_for<FD>([&](auto Q_) { read_k(Q_, I1{}, kf[decltype(Q_)::value % NF]); });
  }

  // ---- the phases.  L is odd: phase 0 (no PV yet), then pairs of full phases (u odd, u + 1 even) while S(u + 2)
  // is still wanted, then this wave's two last phases L (X and PV) and L + 1 (PV), then - while other waves of the
  // workgroup still multiply - phases that only keep up this wave's share of the loads and of the barriers.
  const int nphases = 2 * nblocks + 1;
  phase(I0{}, T{}, T{}, F{}, 0);
  between(0, true);
  int u = 1;
  for (; u + 1 < L; u += 2) {
    if constexpr (MI355_ATTN_PIPE_FUSED_SLOTS) phase_full(I1{}, u); else phase(I1{}, T{}, T{}, T{}, u);
    between(u, true);
    if constexpr (MI355_ATTN_PIPE_FUSED_SLOTS) phase_full(I0{}, u + 1); else phase(I0{}, T{}, T{}, T{}, u + 1);
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
  if constexpr (MI355_ATTN_PIPE_TIMING != 0) {
    if (blockIdx.x == 0 && lane == 0) {
      unsigned long long* dbg = (unsigned long long*)(p.lse + (int64_t)p.Z * p.H * p.N) + wave * 8;   // (behind M: the caller of this experiment makes room)
      for (int i = 0; i < 5; i++) dbg[i] = tsum[i];
    }
  }
#pragma unroll
  for (int i = 0; i < NF; i++) { lds_use(kf[i]); lds_use(vf[i][0]); lds_use(vf[i][1]); }

  // ---- epilogue: O = acc / l, M = m + log2(l); 16 bytes per lane after exchanging register groups 2 a / 2 a + 1
  // between the two lanes of a row (the memory pipeline takes a request per piece whatever its size)
  retire_mfmas();
  retire_mfmas();
#pragma unroll
  for (int b = 0; b < 2; b++) {
    const float l = pair_sum(l_i[b]);
    const int row = row0 + b * 32 + l32;
    const float inv = pend[b] / l;        // (a rescale still pending is applied here)
    if (g == 0) p.lse[(int64_t)hz * p.N + row] = m_i[b] + log2f(l);
    char* dst = obase + (int64_t)row * opitch + g * 16;
#pragma unroll
    for (int c = 0; c < 4; c++) {
      pin_a(oacc[c][b]);
#pragma unroll
      for (int a = 0; a < 2; a++) {
        int x0 = pack2<S>(oacc[c][b][a * 8] * inv, oacc[c][b][a * 8 + 1] * inv);
        int x1 = pack2<S>(oacc[c][b][a * 8 + 2] * inv, oacc[c][b][a * 8 + 3] * inv);
        int y0 = pack2<S>(oacc[c][b][a * 8 + 4] * inv, oacc[c][b][a * 8 + 5] * inv);
        int y1 = pack2<S>(oacc[c][b][a * 8 + 6] * inv, oacc[c][b][a * 8 + 7] * inv);
        swap32_regs(x0, y0);
        swap32_regs(x1, y1);
        *(i32x4*)(dst + (c * 32 + a * 16) * 2) = i32x4{x0, x1, y0, y1};
      }
    }
  }
}

template <typename S, bool BF>
static int launch_fwd_pipe(const AttnArgs& p, hipStream_t stream) {
  constexpr int BM = 256, smem = (3 + 4) * 64 * 256;
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)attn_fwd_pipe_kernel<S, BF>, hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) return (int)e;
    attr_set = true;
  }
  const int nqb = p.N / BM;
  attn_fwd_pipe_kernel<S, BF><<<dim3(nqb * p.Z * p.H), dim3(256), smem, stream>>>(p);
  return (int)hipGetLastError();
}

// head_dim 128, N_CTX a multiple of 256, a positive softmax scale
bool attn_fwd_pipe_ok(const AttnArgs& p) {
  return p.D == 128 && p.d_real == 128 && p.N % 256 == 0 && p.sm_scale > 0.f;
}

int attn_fwd_pipe_launch(const AttnArgs& p, bool bf16, hipStream_t stream) {
  return bf16 ? launch_fwd_pipe<__bf16, true>(p, stream) : launch_fwd_pipe<_Float16, false>(p, stream);
}

}  // namespace mi355

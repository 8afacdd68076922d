// Fused flash-attention forward for fp8 inputs (e5m2 as in the reference, or e4m3fn), head_dim 256, 128
// or 64, and 32 or 16 as a padded form of 64 (python/tutorials/06-fused-attention.py:447 admits these five for every
// type): q, k [Z,H,N,D] with D contiguous, v with N contiguous (the reference transposes V in
// memory for fp8, python/tutorials/06-fused-attention.py:609-614 and :127-135), o in the input
// type, M in fp32.  Same algorithm and rounding points as the 16-bit kernel (attn_fwd.hip): S in
// fp32 from an fp8 x fp8 MFMA, softmax in fp32 in the exp2 domain, P rounded to the fp8 type before
// the second product (`p.to(tl.float8e5)`, :66-67), fp32 accumulator, one rounding of O.
//
// MI355X layout: the 32x32x64 f8f6f4 MFMA wants 32 K-contiguous bytes per lane from both operands.
//   * S^T = K Q^T: the 32 key rows of an MFMA tile are read in a permuted order (tile row
//     8a + 4b + e holds key 16b + 4a + e), so that afterwards the 16 scores a lane holds per tile
//     belong to 16 CONSECUTIVE keys.  P^T, packed four values per register, is then directly the
//     B operand of O^T = V^T P^T with the matching V bytes being two 16-byte pieces of a V^T row.
//   * K tiles [64 keys][D bytes] and V^T tiles [D rows][64 key bytes] go global -> LDS by direct
//     loads into two stages; both are read with ds_read_b128 under XOR swizzles chosen for the
//     64-bank LDS and these access patterns.
#include "common.h"
#include "launch.h"
#include "attn_tiles.h"

namespace mi355 {

template <int FMT>
__device__ __forceinline__ f32x16 mfma_f8(i32x8 a, i32x8 b, f32x16 c) {
#if MI355_DEVICE_PASS
  return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, FMT, FMT, 0, 0, 0, 0);
#else
  return c;
#endif
}

// PAD (D = 64 only): the tensors hold p.d_real = 16 or 32 bytes per row of q, k, o and that many rows of V^T; the
// missing columns are zeros that never exist in memory - the Q fragments are zero-filled in registers, the K / V^T
// tiles in LDS are zeroed once and only the chunks present are ever loaded, and only the first d_real columns of O are
// stored.  Zero columns add nothing to the scores and give zero columns of O: what a HEAD_DIM d_real kernel computes.
template <int FMT, int D, int NW, bool PAD = false>
__global__ __launch_bounds__(NW * 64, NW == 4 && D <= 128 ? 2 : 1) void attn_fwd8_kernel(AttnArgs p) {
  static_assert(!PAD || D == 64, "the padded form is the 64-column one");
  constexpr int BM = NW * 32, BN = 64;
  constexpr int KSQ = D / 64;          // MFMA k-steps of S^T
  constexpr int DT = D / 32;           // 32-row tiles of O^T
  constexpr int KTILE = BN * D;        // K tile: 64 rows of D bytes
  constexpr int VTILE = D * BN;        // V^T tile: D rows of 64 bytes
  constexpr int STAGE = KTILE + VTILE;
  constexpr int KCH = D / 16;          // 16-byte chunks per K row
  constexpr int KINST = KTILE / 1024 / NW, VINST = VTILE / 1024 / NW;
  static_assert(KINST >= 1 && VINST >= 1, "tiles too small for this wave count");

  extern __shared__ __attribute__((aligned(1024))) char smem[];
  LDS_PTR(char) const lds = (LDS_PTR(char))smem;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, g = lane >> 5;

  const int nqb = (p.N + BM - 1) / BM;
  int pid = xcd_remap(blockIdx.x, nqb * p.Z * p.H);
  const int hz = pid / nqb;
  int qb = pid % nqb;
  if (p.causal) qb = nqb - 1 - qb;
  const int z = hz / p.H, h = hz % p.H;
  const int m0 = qb * BM, row0 = m0 + wave * 32;

  const char* qbase = p.q + (int64_t)z * p.sq[0] + (int64_t)h * p.sq[1];
  const char* kbase = p.k + (int64_t)z * p.sk[0] + (int64_t)h * p.sk[1];
  const char* vbase = p.v + (int64_t)z * p.sv[0] + (int64_t)h * p.sv[1];
  char* obase = p.o + (int64_t)z * p.so[0] + (int64_t)h * p.so[1];
  const int64_t qpitch = p.sq[2], kpitch = p.sk[2], vpitch = p.sv[3], opitch = p.so[2];  // bytes: one per element

  // Q operand: lane (query row l32, half g) holds Q[row][64*ks + 32*g .. +32]
  i32x8 qf[KSQ];
  {
    const int r = min(row0 + l32, p.N - 1);
    const char* src = qbase + (int64_t)r * qpitch + g * 32;
#pragma unroll
    for (int ks = 0; ks < KSQ; ks++) {
      i32x4 lo = {0, 0, 0, 0}, hi = {0, 0, 0, 0};
      if (!PAD || ks * 64 + g * 32 < p.d_real) lo = *(const i32x4*)(src + ks * 64);
      if (!PAD || ks * 64 + g * 32 + 16 < p.d_real) hi = *(const i32x4*)(src + ks * 64 + 16);
      qf[ks] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    }
  }

  // swizzles: K rows of D bytes (D = 128: two rows per 256-byte bank sweep, D = 256: one), V^T rows of 64 bytes
  // (a ds_read_b128 is served 16 lanes at a time; with the permuted key order those are key rows
  //  0-7 and 16-23, or 8-15 and 24-31, of a 32-row tile - the XOR value must separate exactly those)
  auto kswz8 = [](int row) {
    return D == 256 ? ((row & 7) | (((row >> 4) & 1) << 3))
         : D == 128 ? (((row >> 1) & 3) | (((row >> 4) & 1) << 2)) : (((row >> 2) & 1) | (((row >> 4) & 1) << 1));
  };
  auto vswz8 = [](int row) { return (row >> 2) & 3; };

  // direct loads: one wave instruction moves 1 KiB = 1024/D K rows or 16 V^T rows
  // (scalar tile base + 32-bit lane offset: the host bounds the row pitches)
  unsigned offK[KINST], offV[VINST];
  bool presentK[KINST], presentV[VINST];
#pragma unroll
  for (int i = 0; i < KINST; i++) {
    const int r = (i * NW + wave) * (1024 / D) + lane / KCH;
    const int chunk = (lane % KCH) ^ kswz8(r);
    offK[i] = (unsigned)(r * kpitch) + (chunk << 4);
    presentK[i] = !PAD || chunk * 16 < p.d_real;
  }
#pragma unroll
  for (int i = 0; i < VINST; i++) {
    const int r = (i * NW + wave) * 16 + lane / 4;   // d row
    offV[i] = (unsigned)(r * vpitch) + (((lane % 4) ^ vswz8(r)) << 4);
    presentV[i] = !PAD || r < p.d_real;
  }
  const unsigned lds_base = lds_addr(lds);
  if constexpr (PAD) {
    lds_zero(lds, 2 * STAGE, tid, NW * 64);
    __syncthreads();
  }
  auto issue_kv = [&](int j, int stage) {
    const unsigned kd = lds_base + stage * STAGE, vd = kd + KTILE;
    const char* ksrc = kbase + (int64_t)j * BN * kpitch;
    const char* vsrc = vbase + (int64_t)j * BN;
#pragma unroll
    for (int i = 0; i < KINST; i++)
      if (presentK[i]) async_copy16_sbase(ksrc, offK[i], kd + (i * NW + wave) * 1024);
#pragma unroll
    for (int i = 0; i < VINST; i++)
      if (presentV[i]) async_copy16_sbase(vsrc, offV[i], vd + (i * NW + wave) * 1024);
  };

  // per-lane LDS offsets.  K operand of tile row l32 = 8a + 4b + e is key row 16b + 4a + e
  // (+32 for the second tile); lane group g feeds bytes 64*ks + 32*g .. +32 as two 16-byte pieces.
  const int krow = ((l32 >> 2) & 1) * 16 + (l32 >> 3) * 4 + (l32 & 3);
  unsigned ka[KSQ][2];
#pragma unroll
  for (int ks = 0; ks < KSQ; ks++)
#pragma unroll
    for (int h2 = 0; h2 < 2; h2++) ka[ks][h2] = krow * D + (((ks * 4 + g * 2 + h2) ^ kswz8(krow)) << 4);
  // V^T operand of O^T rows 32c + l32: lane group g feeds keys 16g .. +16 and 32 + 16g .. +16
  unsigned va[2];
#pragma unroll
  for (int h2 = 0; h2 < 2; h2++) va[h2] = KTILE + l32 * 64 + (((2 * h2 + g) ^ vswz8(l32)) << 4);
  const unsigned lds0 = lds_addr(lds);

  f32x16 oacc[DT];
#pragma unroll
  for (int c = 0; c < DT; c++)
#pragma unroll
    for (int r = 0; r < 16; r++) oacc[c][r] = 0.f;
  float m_i = -INFINITY, l_i = 0.f;

  const float qk_scale = p.sm_scale * 1.44269504f;
  // lazy running maximum, see attn_fwd.hip; P stays below 2^RESCALE_LOG2, far inside both fp8 ranges
  constexpr float RESCALE_LOG2 = 4.f;

  const int kv_end_blk = p.causal ? min(p.N, m0 + BM) : p.N;
  const int nsteps = (kv_end_blk + BN - 1) / BN;
  const int wave_last = p.causal ? (row0 + 31) / BN : nsteps - 1;
  const int wave_first_masked = p.causal ? row0 / BN : nsteps;

  issue_kv(0, 0);
  wait_all();
  __syncthreads();

  auto step = [&](const int j, auto STAGE_) {
    constexpr int SOFF = decltype(STAGE_)::value * STAGE;
    if (j + 1 < nsteps) issue_kv(j + 1, decltype(STAGE_)::value ^ 1);
    if (j <= wave_last && row0 < p.N) {
      const unsigned base = lds0 + SOFF;
      // ---- S^T = K Q^T for the two 32-key tiles
      f32x16 s[2];
      {
        i32x4 kf[2][KSQ][2];
        static_for<2>([&](auto A_) {
          constexpr int a = decltype(A_)::value;
          static_for<KSQ>([&](auto KS_) {
            constexpr int ks = decltype(KS_)::value;
            kf[a][ks][0] = lds_read_b128<a * 32 * D>(base + ka[ks][0]);
            kf[a][ks][1] = lds_read_b128<a * 32 * D>(base + ka[ks][1]);
          });
        });
        static_for<2>([&](auto A_) {
          constexpr int a = decltype(A_)::value;
          lds_wait<(1 - a) * 2 * KSQ>();
          static_for<KSQ>([&](auto KS_) {
            constexpr int ks = decltype(KS_)::value;
            lds_use(kf[a][ks][0]);
            lds_use(kf[a][ks][1]);
            i32x8 kop = __builtin_shufflevector(kf[a][ks][0], kf[a][ks][1], 0, 1, 2, 3, 4, 5, 6, 7);
            if constexpr (ks == 0) {
              f32x16 zero;
#pragma unroll
              for (int r = 0; r < 16; r++) zero[r] = 0.f;
              s[a] = mfma_f8<FMT>(kop, qf[0], zero);
            } else {
              s[a] = mfma_f8<FMT>(kop, qf[ks], s[a]);
            }
          });
        });
      }
      // V^T operands of the first O^T tiles while the softmax runs
      i32x4 vf[DT][2];
      static_for<DT>([&](auto C_) {
        constexpr int c = decltype(C_)::value;
        vf[c][0] = lds_read_b128<c * 32 * 64>(base + va[0]);
        vf[c][1] = lds_read_b128<c * 32 * 64>(base + va[1]);
      });
      // ---- online softmax; register r of tile a is key 32a + 16g + r of this lane's query row
      if (j >= wave_first_masked) {
        const int qrow = row0 + l32;
#pragma unroll
        for (int a = 0; a < 2; a++)
#pragma unroll
          for (int r = 0; r < 16; r++)
            if (j * BN + a * 32 + g * 16 + r > qrow) s[a][r] = -INFINITY;
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
      float rs = 0.f;
#pragma unroll
      for (int a = 0; a < 2; a++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
          float pv = fast_exp2(fmaf(s[a][r], qk_scale, -m_i));
          s[a][r] = pv;
          rs += pv;
        }
      l_i += rs;
      i32x8 pop;  // P^T operand: bytes 0..15 = tile 0 (keys 16g..), bytes 16..31 = tile 1 (keys 32 + 16g..)
#pragma unroll
      for (int a = 0; a < 2; a++)
#pragma unroll
        for (int w = 0; w < 4; w++)
          pop[a * 4 + w] = pack4_fp8<FMT>(s[a][4 * w], s[a][4 * w + 1], s[a][4 * w + 2], s[a][4 * w + 3]);
      // ---- O^T += V^T P^T
      lds_wait<0>();
      static_for<DT>([&](auto C_) {
        constexpr int c = decltype(C_)::value;
        lds_use(vf[c][0]);
        lds_use(vf[c][1]);
        i32x8 vop = __builtin_shufflevector(vf[c][0], vf[c][1], 0, 1, 2, 3, 4, 5, 6, 7);
        oacc[c] = mfma_f8<FMT>(vop, pop, oacc[c]);
      });
    }
    wait_all();
    __syncthreads();
  };

  for (int j = 0; j < nsteps; j += 2) {
    step(j, std::integral_constant<int, 0>{});
    if (j + 1 < nsteps) step(j + 1, std::integral_constant<int, 1>{});
  }

  // ---- epilogue: O = acc / l rounded to the fp8 type, M = m + log2(l)
  {
    const float l = pair_sum(l_i);
    const int row = row0 + l32;
    if (row0 < p.N) {   // (wave-uniform: N is a multiple of 32)
      const float inv = 1.f / l;
      if (g == 0) p.lse[(int64_t)hz * p.N + row] = m_i + log2f(l);
      // A lane owns one dword (4 codes) per register group: dwords 0, 2, 4, 6 of a tile's 32-byte row segment in lane
      // l32, dwords 1, 3, 5, 7 in lane l32 + 32.  Two exchanges between the lanes of a row (v_permlane32_swap: the
      // upper half of the first register with the lower half of the second) give lane l32 the dwords 0 .. 3 and lane
      // l32 + 32 the dwords 4 .. 7: one store of 16 bytes per tile instead of four of 4 bytes - the memory pipeline
      // takes a request per piece.
      char* dst = obase + (int64_t)row * opitch + g * 16;
#pragma unroll
      for (int c = 0; c < DT; c++) {
        int w[4];
#pragma unroll
        for (int rg = 0; rg < 4; rg++)
          w[rg] = pack4_fp8<FMT>(oacc[c][rg * 4] * inv, oacc[c][rg * 4 + 1] * inv, oacc[c][rg * 4 + 2] * inv, oacc[c][rg * 4 + 3] * inv);
        swap32_regs(w[0], w[2]);
        swap32_regs(w[1], w[3]);
        if (!PAD || c * 32 + g * 16 < p.d_real) *(i32x4*)(dst + c * 32) = i32x4{w[0], w[2], w[1], w[3]};
      }
    }
  }
}

template <int FMT, int D, int NW, bool PAD = false>
static int launch_fwd8(const AttnArgs& p, hipStream_t stream) {
  constexpr int BM = NW * 32;
  constexpr int smem = 2 * 2 * 64 * D;
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)attn_fwd8_kernel<FMT, D, NW, PAD>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    if (e != hipSuccess) return (int)e;
    attr_set = true;
  }
  const int nqb = (p.N + BM - 1) / BM;
  attn_fwd8_kernel<FMT, D, NW, PAD><<<dim3(nqb * p.Z * p.H), dim3(NW * 64), smem, stream>>>(p);
  return (int)hipGetLastError();
}

template <int FMT>
static int launch_fwd8_fmt(const AttnArgs& p, hipStream_t stream) {
  // variant 2: eight waves (256 query rows per K/V stream), head_dim 128 only
  if (p.D == 256) return launch_fwd8<FMT, 256, 4>(p, stream);   // (one workgroup per CU: 128 accumulator registers per lane)
  if (p.D == 128) return p.variant == 2 ? launch_fwd8<FMT, 128, 8>(p, stream) : launch_fwd8<FMT, 128, 4>(p, stream);
  if (p.d_real < p.D) return launch_fwd8<FMT, 64, 4, true>(p, stream);    // head dims 16 / 32
  return launch_fwd8<FMT, 64, 4>(p, stream);
}

int attn_fwd8_launch(const AttnArgs& p, bool e5m2, hipStream_t stream) {
  return e5m2 ? launch_fwd8_fmt<1>(p, stream) : launch_fwd8_fmt<0>(p, stream);
}

}  // namespace mi355

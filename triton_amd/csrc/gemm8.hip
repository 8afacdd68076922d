// fp8 (e4m3fn / e5m2) instantiation of the tiled MFMA GEMM core: 64 elements per K step, one
// 32x32x64 f8f6f4 MFMA sub-step (large products with whole tiles run the four-wave kernel of gemm_wave128.hip instead,
// either B layout).  Every kernel form here takes both operands K-major (the layout the reference uses
// for fp8: `matmul(a, b.T)` with b stored [N, K], python/tutorials/03-matrix-multiplication.py:378-382,
// python/tutorials/09-persistent-matmul.py:396-407); a row-major B[K, N] (what `matmul(a, b)` passes without that
// host-side transpose) runs the one-barrier-per-step form, which transposes it on its way out of LDS.
#include "gemm_core.h"
#include "formats.h"

namespace mi355 {

template <int FMT>  // 0 = e4m3fn, 1 = e5m2 (cbsz / blgp encoding of the instruction)
struct Cfg8 {
  using Operand = i32x8;
  static constexpr int kSteps = 1, kChunks = 2;
  static constexpr bool kRowMajorB = true, kScaled = false;   // (row-major B: the one-barrier-per-step kernel only)
  static constexpr int kElemBytes = 1;
  static constexpr int kStepsPerScaleDword = 1;
  // no block scales: placeholders so that generic code naming them compiles
  __device__ static int scale_dword_offset(int) { return 0; }
  __device__ static int scale_fixup(int v, int, int) { return v; }
  // A lane feeds 32 bytes per sub-step as two 16-byte halves; any assignment of K positions
  // works as long as both operands use the same one.
  __device__ static constexpr int chunk(int, int g, int c) { return c * 2 + g; }
  template <int ks>
  __device__ static f32x16 mma(Operand a, Operand b, f32x16 c, int, int) {
#if MI355_DEVICE_PASS
    return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, FMT, FMT, 0, 0, 0, 0);
#else
    return c;
#endif
  }
};

// ---------------------------------------------------------------------------------------------
// Skinny fp8 GEMM (M <= 32, the decode shape): the work is reading B once, so there is no tile
// reuse to organise - one workgroup per 32 columns of C, its four waves split K, every lane
// streams whole 128-byte pieces of its B row (K-major) straight into MFMA operand registers, and
// the partial 32x32 accumulators meet in LDS at the end.  A (at most 32 x K bytes) is
// re-read by every workgroup from L2.  Lane (row l%32, half l/32) of K chunk c feeds bytes
// 256 c + 128 (l/32) + 32 s .. + 32 of its row into sub-step s = 0..3; A uses the same
// assignment, which is all the MFMA needs.
// ---------------------------------------------------------------------------------------------
template <int FMT>
__global__ __launch_bounds__(256) void gemm8_skinny_kernel(GemmArgs p) {
  constexpr int CH = 256;  // bytes of K per chunk
  constexpr int NW = 4;    // waves that split K
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, g = lane >> 5;
  const int n0 = blockIdx.x * 32;
  const int nchunks = p.k_bytes / CH;
  const char* arow = p.A + (int64_t)min(l32, p.M - 1) * p.lda + g * 128;
  const char* brow = p.B + (int64_t)min(n0 + l32, p.N - 1) * p.ldb + g * 128;

  f32x16 acc;
#pragma unroll
  for (int r = 0; r < 16; r++) acc[r] = 0.f;

  i32x4 fa[2][8], fb[2][8];
  auto load_chunk = [&](int c, int set) {
#pragma unroll
    for (int i = 0; i < 8; i++) {
      fb[set][i] = *(const i32x4*)(brow + (int64_t)c * CH + i * 16);
      fa[set][i] = *(const i32x4*)(arow + (int64_t)c * CH + i * 16);
    }
  };
  auto mma_chunk = [&](int set) {
#pragma unroll
    for (int s4 = 0; s4 < 4; s4++) {
      i32x8 a = __builtin_shufflevector(fa[set][2 * s4], fa[set][2 * s4 + 1], 0, 1, 2, 3, 4, 5, 6, 7);
      i32x8 b = __builtin_shufflevector(fb[set][2 * s4], fb[set][2 * s4 + 1], 0, 1, 2, 3, 4, 5, 6, 7);
#if MI355_DEVICE_PASS
      // D[m][n]: lane owns column n = l%32 of 16 rows m
      acc = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, acc, FMT, FMT, 0, 0, 0, 0);
#endif
    }
  };
  // every wave takes a contiguous share of the chunks (each lane then walks its row in
  // consecutive 256-byte strides), the next chunk's loads in flight during the MFMAs
  const int per = (nchunks + NW - 1) / NW;
  const int cend = min(nchunks, (wave + 1) * per);
  int c = wave * per;
  if (c < cend) load_chunk(c, 0);
  for (; c < cend; c += 2) {
    if (c + 1 < cend) load_chunk(c + 1, 1);
    mma_chunk(0);
    if (c + 1 < cend) {
      if (c + 2 < cend) load_chunk(c + 2, 0);
      mma_chunk(1);
    }
  }

  // reduce the partial accumulators through LDS: red[wave][r][lane]
  __shared__ float red[NW][16][64];
#pragma unroll
  for (int r = 0; r < 16; r++) red[wave][r][lane] = acc[r];
  __syncthreads();
  float alpha = 1.f;
  if (p.a_scale) alpha *= *p.a_scale;
  if (p.b_scale) alpha *= *p.b_scale;
  // wave w finishes registers 2w, 2w+1: rows m = 8*(r/4) + 4*g + (r%4), column n0 + l32
#pragma unroll
  for (int e = 0; e < 16 / NW; e++) {
    const int r = wave * (16 / NW) + e;
    float v = 0.f;
#pragma unroll
    for (int w = 0; w < NW; w++) v += red[w][r][lane];
    v *= alpha;
    if (p.activation == 1) v = v >= 0.f ? v : 0.01f * v;
    const int m = (r >> 2) * 8 + g * 4 + (r & 3), n = n0 + l32;
    if (m < p.M && n < p.N) {
      const int64_t off = (int64_t)m * p.ldc + (int64_t)n * p.scn;
      if (p.out_dtype == 4) ((float*)p.C)[off] = v;
      else if (p.out_dtype == 2) ((uint8_t*)p.C)[off] = f32_to_e4m3(v);
      else if (p.out_dtype == 3) ((uint8_t*)p.C)[off] = f32_to_e5m2(v);
      else if (p.out_dtype == 1) ((__bf16*)p.C)[off] = (__bf16)v;
      else ((_Float16*)p.C)[off] = (_Float16)v;
    }
  }
}

bool gemm8_skinny_ok(const GemmArgs& p) { return p.M <= 32 && p.k_bytes >= 256 && p.k_bytes % 256 == 0; }

int gemm8_skinny_launch(const GemmArgs& p, bool e5m2, hipStream_t stream) {
  dim3 grid((p.N + 31) / 32), block(256);
  if (e5m2) gemm8_skinny_kernel<1><<<grid, block, 0, stream>>>(p);
  else gemm8_skinny_kernel<0><<<grid, block, 0, stream>>>(p);
  return (int)hipGetLastError();
}

int gemm8_launch(const GemmArgs& p, bool e5m2, bool b_kmajor, int tile, hipStream_t stream) {
  if (!b_kmajor) {
    // 128x128 tiles (two workgroups per CU) where the dispatcher chose them, 256x256 tiles otherwise
    if (tile == 1) return e5m2 ? launch_gemm<Cfg8<1>, 128, 128, 2, 2, false, 4>(p, stream) : launch_gemm<Cfg8<0>, 128, 128, 2, 2, false, 4>(p, stream);
    return e5m2 ? launch_gemm<Cfg8<1>, 256, 256, 2, 4, false, 4>(p, stream) : launch_gemm<Cfg8<0>, 256, 256, 2, 4, false, 4>(p, stream);
  }
  return e5m2 ? launch_gemm_tile<Cfg8<1>, true>(p, tile, stream) : launch_gemm_tile<Cfg8<0>, true>(p, tile, stream);
}

int gemm8_splitk_launch(const GemmArgs& p, bool e5m2, bool b_kmajor, int splits, int chunk_bytes, hipStream_t stream) {
  if (b_kmajor) return e5m2 ? launch_gemm_splitk<Cfg8<1>, true>(p, splits, chunk_bytes, stream) : launch_gemm_splitk<Cfg8<0>, true>(p, splits, chunk_bytes, stream);
  return e5m2 ? launch_gemm_splitk<Cfg8<1>, false>(p, splits, chunk_bytes, stream) : launch_gemm_splitk<Cfg8<0>, false>(p, splits, chunk_bytes, stream);
}

}  // namespace mi355

// fp16 / bf16 instantiation of the tiled MFMA GEMM core: 32 elements (64 bytes) per K step,
// two 32x32x16 MFMA sub-steps, row-major or K-major B.
#include "gemm_core.h"

namespace mi355 {

template <typename V8>
struct Cfg16 {
  using Operand = V8;
  static constexpr int kSteps = 2, kChunks = 1;
  static constexpr bool kRowMajorB = true, kScaled = false;
  static constexpr int kElemBytes = 2;
  static constexpr int kStepsPerScaleDword = 1;
  // no block scales: placeholders so that generic code naming them compiles
  __device__ static int scale_dword_offset(int) { return 0; }
  __device__ static int scale_fixup(int v, int, int) { return v; }
  // lane group g of sub-step ks reads k elements 16*ks + 8*g .. +8
  __device__ static constexpr int chunk(int ks, int g, int) { return ks * 2 + g; }
  template <int ks>
  __device__ static f32x16 mma(Operand a, Operand b, f32x16 c, int, int) { return mfma32(a, b, c); }
};

int gemm16_launch(const GemmArgs& p, bool bf16, bool b_kmajor, int tile, hipStream_t stream) {
  if (bf16) {
    return b_kmajor ? launch_gemm_tile<Cfg16<bf16x8>, true>(p, tile, stream)
                    : launch_gemm_tile<Cfg16<bf16x8>, false>(p, tile, stream);
  }
  return b_kmajor ? launch_gemm_tile<Cfg16<f16x8>, true>(p, tile, stream)
                  : launch_gemm_tile<Cfg16<f16x8>, false>(p, tile, stream);
}

int gemm16_splitk_launch(const GemmArgs& p, bool bf16, bool b_kmajor, int splits, int chunk_bytes, hipStream_t stream) {
  if (bf16) {
    return b_kmajor ? launch_gemm_splitk<Cfg16<bf16x8>, true>(p, splits, chunk_bytes, stream)
                    : launch_gemm_splitk<Cfg16<bf16x8>, false>(p, splits, chunk_bytes, stream);
  }
  return b_kmajor ? launch_gemm_splitk<Cfg16<f16x8>, true>(p, splits, chunk_bytes, stream)
                  : launch_gemm_splitk<Cfg16<f16x8>, false>(p, splits, chunk_bytes, stream);
}

int gemm16_grouped_launch(const GroupedArgs& ga, bool bf16, int nprog, int nprog_big, hipStream_t stream) {
  return bf16 ? launch_gemm_grouped<Cfg16<bf16x8>, __bf16>(ga, nprog, nprog_big, stream)
              : launch_gemm_grouped<Cfg16<f16x8>, _Float16>(ga, nprog, nprog_big, stream);
}

}  // namespace mi355

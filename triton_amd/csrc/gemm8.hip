// fp8 (e4m3fn / e5m2) instantiation of the tiled MFMA GEMM core: 64 elements per K step, one
// 32x32x64 f8f6f4 MFMA sub-step, both operands K-major (the layout the reference uses for fp8:
// `matmul(a, b.T)` with b stored [N, K], python/tutorials/03-matrix-multiplication.py:378-382,
// python/tutorials/09-persistent-matmul.py:396-407).
#include "gemm_core.h"

namespace mi355 {

template <int FMT>  // 0 = e4m3fn, 1 = e5m2 (cbsz / blgp encoding of the instruction)
struct Cfg8 {
  using Operand = i32x8;
  static constexpr int kSteps = 1, kChunks = 2;
  static constexpr bool kRowMajorB = false, kScaled = false;
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

int gemm8_launch(const GemmArgs& p, bool e5m2, int tile, hipStream_t stream) {
  return e5m2 ? launch_gemm_tile<Cfg8<1>, true>(p, tile, stream) : launch_gemm_tile<Cfg8<0>, true>(p, tile, stream);
}

}  // namespace mi355

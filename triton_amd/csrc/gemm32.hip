// fp32 instantiation of the tiled MFMA GEMM core: fp32 operands on the fp32 MFMAs (v_mfma_f32_32x32x2_f32: exact fp32
// products, fp32 accumulation - the `ieee` input precision of `tl.dot`, which is what the reference's CPU path computes
// for fp32 operands: python/triton/runtime/interpreter.py:542-549, np.matmul in fp32).  A K step is the 64 bytes of
// every operand row of the other types, here 16 elements: a lane's 16-byte chunk feeds four MFMAs of two k each (lane
// group g supplies k = g of an MFMA; which element of the row that is is free as long as A and B agree: chunk 2 ks + g,
// element j, for MFMA j of sub-step ks).  K-major B only - the LDS transpose reads exist for 16-, 8-, 6- and 4-bit
// elements -; a row-major B is put K-major by the host wrapper or runs the any-stride kernel.
#include "gemm_core.h"

namespace mi355 {

struct Cfg32 {
  using Operand = f32x4;
  static constexpr int kSteps = 2, kChunks = 1;
  static constexpr bool kRowMajorB = false, kScaled = false;
  static constexpr int kElemBytes = 4;
  static constexpr int kStepsPerScaleDword = 1;
  __device__ static int scale_dword_offset(int) { return 0; }
  __device__ static int scale_fixup(int v, int, int) { return v; }
  __device__ static constexpr int chunk(int ks, int g, int) { return ks * 2 + g; }
  template <int ks>
  __device__ static f32x16 mma(Operand a, Operand b, f32x16 c, int, int) {
#if MI355_DEVICE_PASS
#pragma unroll
    for (int j = 0; j < 4; j++) c = __builtin_amdgcn_mfma_f32_32x32x2f32(a[j], b[j], c, 0, 0, 0);
#endif
    return c;
  }
};

// tile: as for the other types' tile kernels (launch_gemm_tile: 1 = 128x128 tiles, 2 = 256x256 with one barrier per K
// step, 4 = software pipelined, 5 = its persistent form)
int gemm32_launch(const GemmArgs& p, int tile, hipStream_t stream) {
  return launch_gemm_tile<Cfg32, true>(p, tile, stream);
}

int gemm32_splitk_launch(const GemmArgs& p, int splits, int chunk_bytes, hipStream_t stream) {
  return launch_gemm_splitk<Cfg32, true>(p, splits, chunk_bytes, stream);
}

}  // namespace mi355

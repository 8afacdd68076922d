// Block-scaled (OCP MX v1.0) instantiations of the tiled MFMA GEMM core: MXFP4 (e2m1, 128
// elements per 64-byte K step, two 32x32x64 sub-steps) and MXFP8 (e4m3, 64 elements, one
// sub-step), one e8m0 scale per 32 elements of K applied inside the MFMA.
//
// How the scaled 32x32x64 f8f6f4 MFMA takes its scales (measured on gfx950): every lane passes
// one dword and a byte selector.  fp4: the selected byte of lane (row, g) scales that lane's own
// 32 elements.  fp8: registers 0-3 of both lane groups form K block 0 and are scaled by the byte
// from lane group 0, registers 4-7 form K block 1 and take the byte from lane group 1.  The K
// positions a lane reads are therefore chosen such that the scale byte it needs sits at a byte
// position that does not depend on the lane.
#include "gemm_core.h"
#include "formats.h"

namespace mi355 {

struct CfgMxfp4 {
  using Operand = i32x4;
  static constexpr int kSteps = 2, kChunks = 1;
  static constexpr int kStepsPerScaleDword = 1;  // 4 scale bytes per row and K step
  static constexpr bool kRowMajorB = false, kScaled = true;
  static constexpr int kElemBytes = 1;
  // lane group g reads scale blocks 2g, 2g+1 of the step (16 bytes = 32 elements each), one per sub-step
  __device__ static constexpr int chunk(int ks, int g, int) { return g * 2 + ks; }
  // the step has 4 scale bytes per row; move bytes 2g, 2g+1 to positions 0, 1 (selector = ks)
  // (scale rows of any pitch: the four bytes need not be aligned - the compiler emits what the target allows)
  __device__ static int load_scale(const uint8_t* row, int kt, int g) {
    uint32_t v;
    __builtin_memcpy(&v, row + kt * 4, 4);
    return (int)(v >> (16 * g));
  }
  // the last, partial step: `nblocks` (1 .. 3) scale bytes exist; the others become 2^0, next to zero-filled operands
  __device__ static int load_scale_tail(const uint8_t* row, int kt, int g, int nblocks) {
    uint32_t v = 0x7F7F7F7Fu;
#pragma unroll
    for (int i = 0; i < 4; i++)
      if (i < nblocks) v = (v & ~(0xFFu << (8 * i))) | ((uint32_t)row[kt * 4 + i] << (8 * i));
    return (int)(v >> (16 * g));
  }
  static constexpr int kBlockBytes = 16;   // operand bytes per scale block
  __device__ static int scale_dword_offset(int kt) { return kt * 4; }          // dword copied to LDS for step kt
  __device__ static int scale_fixup(int v, int, int g) { return (int)((unsigned)v >> (16 * g)); }
  template <int ks>
  __device__ static f32x16 mma(Operand a, Operand b, f32x16 c, int sa, int sb) {
#if MI355_DEVICE_PASS
    // fp4 operands occupy the low four registers; the high four are not read by the hardware
    i32x8 a8 = __builtin_shufflevector(a, a, 0, 1, 2, 3, -1, -1, -1, -1);
    i32x8 b8 = __builtin_shufflevector(b, b, 0, 1, 2, 3, -1, -1, -1, -1);
    return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a8, b8, c, 4, 4, ks, sa, ks, sb);
#else
    return c;
#endif
  }
};

struct CfgMxfp8 {
  using Operand = i32x8;
  static constexpr int kSteps = 1, kChunks = 2;
  static constexpr int kStepsPerScaleDword = 2;  // 2 scale bytes per row and K step
  static constexpr bool kRowMajorB = false, kScaled = true;
  static constexpr int kElemBytes = 1;
  // register half c is scale block c of the step; lane group g holds its 16-byte half g
  __device__ static constexpr int chunk(int, int g, int c) { return 2 * c + g; }
  // the step has 2 scale bytes per row; lane group g supplies the scale of block g in byte 0
  __device__ static int load_scale(const uint8_t* row, int kt, int g) {
    uint16_t v;
    __builtin_memcpy(&v, row + kt * 2, 2);
    return (int)v >> (8 * g);
  }
  // the last, partial step holds one scale block; the other becomes 2^0, next to zero-filled operands
  __device__ static int load_scale_tail(const uint8_t* row, int kt, int g, int) {
    return (int)((uint32_t)row[kt * 2] | 0x7F00u) >> (8 * g);
  }
  static constexpr int kBlockBytes = 32;   // operand bytes per scale block
  // the dword holding the scales of steps kt and kt^1; bytes 2*(kt&1) + g
  __device__ static int scale_dword_offset(int kt) { return (kt >> 1) * 4; }
  __device__ static int scale_fixup(int v, int kt, int g) { return (int)((unsigned)v >> (16 * (kt & 1) + 8 * g)); }
  template <int ks>
  __device__ static f32x16 mma(Operand a, Operand b, f32x16 c, int sa, int sb) {
#if MI355_DEVICE_PASS
    return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, 0, 0, 0, sa, 0, sb);
#else
    return c;
#endif
  }
};

// Any shape / pitch: one thread per output, decode-and-FMA in fp32.  Runs only on request (a negative tile number):
// an independent second implementation for the tests.
__global__ __launch_bounds__(256) void mx_gemm_simple_kernel(GemmArgs p, int fp4) {
  int n = blockIdx.x * 16 + threadIdx.x % 16, m = blockIdx.y * 16 + threadIdx.x / 16;
  if (m >= p.M || n >= p.N) return;
  const uint8_t* a = (const uint8_t*)p.A + (int64_t)m * p.lda;
  const uint8_t* b = (const uint8_t*)p.B + (int64_t)n * p.ldb;
  const uint8_t* sa = p.sA + (int64_t)m * p.lds_a;
  const uint8_t* sb = p.sB + (int64_t)n * p.lds_b;
  float acc = 0.f;
  for (int kb = 0; kb < p.K / 32; kb++) {
    float part = 0.f;
    for (int e = 0; e < 32; e++) {
      int k = kb * 32 + e;
      float x, y;
      if (fp4) {
        x = e2m1_to_f32((a[k >> 1] >> ((k & 1) * 4)) & 15);
        y = e2m1_to_f32((b[k >> 1] >> ((k & 1) * 4)) & 15);
      } else {
        x = e4m3_to_f32(a[k]);
        y = e4m3_to_f32(b[k]);
      }
      part = fmaf(x, y, part);
    }
    acc += part * e8m0_to_f32(sa[kb]) * e8m0_to_f32(sb[kb]);
  }
  int64_t idx = (int64_t)m * p.ldc + n;
  if (p.out_dtype == 4) ((float*)p.C)[idx] = acc;
  else if (p.out_dtype == 1) ((__bf16*)p.C)[idx] = (__bf16)acc;
  else ((_Float16*)p.C)[idx] = (_Float16)acc;
}

int mx_gemm_launch(const GemmArgs& p, int fmt, int tile, hipStream_t stream) {
  // 6: four waves of scaled 16x16x128 MFMAs (whole 256x256 tiles, K at least 1024, any multiple of the scale block:
  // what is left behind the last whole group of K steps is the tail form's)
  if (tile == 6 && fmt == 0 && (p.tile_m == 192 || p.tile_m == 128 || gemm_wave128_mxfp4_ok(p))) return gemm_wave128_mxfp4_launch(p, stream);
  if (tile == 6 && fmt != 0 && (p.tile_m == 192 || p.tile_m == 128 || gemm_wave128_mxfp8_ok(p))) return gemm_wave128_mxfp8_launch(p, stream);
  if (tile < 0) {
    dim3 grid((p.N + 15) / 16, (p.M + 15) / 16);
    mx_gemm_simple_kernel<<<grid, dim3(256), 0, stream>>>(p, fmt == 0);
    return (int)hipGetLastError();
  }
  // K not a whole number of 64-byte steps, or scale rows that are not dword aligned (a contiguous scale matrix whose
  // K / 32 is not a multiple of four): the one-barrier-per-step kernels, which read their scales with loads of any
  // alignment and finish a partial last step themselves
  const bool whole_tiles = p.k_bytes % RBK == 0;
  const bool scales_aligned = p.lds_a % 4 == 0 && p.lds_b % 4 == 0 && ((uintptr_t)p.sA % 4) == 0 && ((uintptr_t)p.sB % 4) == 0;
  if (!whole_tiles || !scales_aligned) tile = tile == 1 ? 1 : 2;
  return fmt == 0 ? launch_gemm_tile<CfgMxfp4, true>(p, tile, stream) : launch_gemm_tile<CfgMxfp8, true>(p, tile, stream);
}

}  // namespace mi355

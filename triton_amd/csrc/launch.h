// Host-side argument blocks and launcher prototypes shared by the kernel files and the C ABI.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mi355 {

struct GemmArgs {
  const char* A;  // [M,K], K-contiguous on the MFMA paths
  const char* B;  // [K,N] (N- or K-contiguous)
  char* C;        // [M,N]
  int M, N, K;
  int k_bytes;    // bytes of one operand row along K (K * element size, K / 2 for fp4)
  int64_t lda;    // MFMA paths: row pitch of A in BYTES
  int64_t ldb;    // MFMA paths: pitch in BYTES between consecutive k rows (row-major B) or n rows (K-major B)
  int64_t ldc;    // elements between consecutive C rows
  int64_t scn;    // elements between consecutive C columns
  const float* a_scale;
  const float* b_scale;
  int activation;
  int out_dtype;  // MI355_F16 / MI355_BF16 / MI355_F32 (fp8 kernels also MI355_F8E4M3)
  int group_m;
  int num_programs;  // persistent kernels: workgroups to launch (0 = not persistent)
  float* workspace;  // stream-K: 2 * num_programs tiles of 256x256 fp32 (NULL = no stream-K)
  int c_vec_ok;   // scn == 1 and every C row start is 16-byte aligned
  int tile_m;     // four-wave 16-bit kernel: 0 / 256 = tiles of 256 x 256, 192 = tiles of 192 x 256
  int lean_ok;    // the four-wave kernels may take their lean epilogue (tuning knob MI355_GEMM_LEAN_EPILOGUE, default 1)
  // optional addend of the epilogue: acc * alpha + aux[m * aux_sm + n * aux_sn] (a zero stride broadcasts
  // a row or a column vector), added in fp32 before the activation; NULL = none
  const void* aux;
  int64_t aux_sm, aux_sn;  // element strides
  int aux_dtype;           // MI355_F16 / MI355_BF16 / MI355_F32
  // block-scaled (MX) kernels only: e8m0 scale matrices [M, K/32], [N, K/32] and their row pitches
  const uint8_t* sA;
  const uint8_t* sB;
  int64_t lds_a, lds_b;
};

// generic strided kernel: strides in elements, any dtype the ABI knows
struct GemmStridedArgs {
  const void* A; const void* B; void* C;
  int M, N, K;
  int64_t sam, sak, sbk, sbn, scm, scn;
  const float* a_scale; const float* b_scale;
  int activation, in_dtype, out_dtype;
  const void* aux; int64_t aux_sm, aux_sn; int aux_dtype;  // as in GemmArgs
};

// skinny GEMM, out[s][l] = sum_k X[s][k] * Y[l][k]
struct SkinnyArgs {
  const char* X;    // small operand: S <= 64 rows, K contiguous or S contiguous
  const char* Y;    // streamed operand: L rows, K contiguous or L contiguous
  char* C;
  int S, L, K;
  int64_t x_pitch;  // bytes between rows s (K contiguous) or between k rows (S contiguous)
  int64_t y_pitch;  // bytes between rows l (K contiguous) or between k rows (L contiguous)
  int64_t cs, cl;   // element strides of the output along s and l
  const float* a_scale;
  const float* b_scale;
  int activation;
  int out_dtype;
  // optional addend of the epilogue, indexed like the output: aux[s * aux_ss + l * aux_sl] (a zero stride
  // broadcasts), added in fp32 before the activation; NULL = none
  const void* aux;
  int64_t aux_ss, aux_sl;
  int aux_dtype;
  int cus;          // compute units of the device (0 = unknown): picks the workgroup width for an L-contiguous Y
};

// one-launch GEMM with row-wise epilogues (row softmax, chained product), N <= 256 and N2 <= 256
struct RowFusedArgs {
  const void* A; const void* B; void* C;
  const void* W;                       // [N, N2] of the chained product, NULL = none
  int M, N, K, N2;
  int64_t sam, sak, sbk, sbn, swn, swn2, scm, scn;   // element strides
  const float* a_scale; const float* b_scale;
  int activation, softmax, out_dtype;
  const void* aux; int64_t aux_sm, aux_sn; int aux_dtype;   // addend as in GemmArgs
};

struct AttnArgs {
  const char* q; const char* k; const char* v; char* o; float* lse;
  const char* d_o; const float* delta; char* dq; char* dk; char* dv;
  int Z, H, N, D;
  int64_t sq[4], sk[4], sv[4], so[4];  // element strides
  float sm_scale;
  int causal;
  int variant;  // tiling variant (tuning knob)
  int num_programs;  // persistent forward: CUs to fill (0 = one workgroup per item)
  int d_real;   // head dims 16 / 32: columns present in memory (D is then 64: the kernels pad with zeros on the fly)
};

// Device-side tables of a grouped GEMM (layout of python/tutorials/08-grouped-gemm.py:66-77).
struct GroupedArgs {
  const uint64_t* a_ptrs;  // [group_size] device addresses
  const uint64_t* b_ptrs;
  const uint64_t* c_ptrs;
  const int* sizes;        // [group_size][3] = M, N, K
  const int* lds;          // [group_size][3] = lda, ldb, ldc in elements
  int group_size;
  int out_dtype;           // element type of A, B and C: 0 = fp16, 1 = bf16
  int big_tiles_min;       // 256x256 tiles in the group from which the large-tile kernel takes the launch
  int chunk;               // four-wave kernel: most consecutive tiles that a program takes as one run (1 = every nprog-th tile)
  int wave128_min_k;       // groups of whole 256x256 tiles with every K >= this go to the four-wave 16x16-MFMA kernel (0 = never)
};

int gemm_wave128_grouped_launch(const GroupedArgs& ga, bool bf16, int nprog, hipStream_t stream);

int gemm16_grouped_launch(const GroupedArgs& ga, bool bf16, int nprog, int nprog_big, hipStream_t stream);
int gemm16_launch(const GemmArgs& p, bool bf16, bool b_kmajor, int tile, hipStream_t stream);
int gemm8_launch(const GemmArgs& p, bool e5m2, bool b_kmajor, int tile, hipStream_t stream);
int gemm32_launch(const GemmArgs& p, int tile, hipStream_t stream);   // fp32 operands, K-major B; tile as for gemm16_launch
// split-K on 128x128 tiles: `splits` chunks of `chunk_bytes` of every operand row (whole K steps of 64 bytes), fp32
// partial tiles into p.workspace ([splits][M][N]); splitk_reduce_launch adds them up and does the epilogue
int gemm16_splitk_launch(const GemmArgs& p, bool bf16, bool b_kmajor, int splits, int chunk_bytes, hipStream_t stream);
int gemm8_splitk_launch(const GemmArgs& p, bool e5m2, bool b_kmajor, int splits, int chunk_bytes, hipStream_t stream);
int gemm32_splitk_launch(const GemmArgs& p, int splits, int chunk_bytes, hipStream_t stream);   // fp32 operands, K-major B
int splitk_reduce_launch(const GemmStridedArgs& out, const float* workspace, int splits, hipStream_t stream);   // A, B, K, in_dtype of `out` unused
bool gemm_wave128_192_ok(const GemmArgs& p, bool b_kmajor, int in_dtype, int tile_m = 192);   // the same for tiles of 192 x 256 / 128 x 256
bool gemm_wave128_ok(const GemmArgs& p, bool b_kmajor, int in_dtype);
bool gemm_wave128_f8_ok(const GemmArgs& p, bool b_kmajor);
bool gemm_wave128_mixed_ok(const GemmArgs& p, bool b_kmajor, int in_dtype, int rows256);   // rows256 rows on 256-row tiles, the rest on 192-row tiles
int gemm_wave128_mixed_launch(const GemmArgs& p, int rows256, bool bf16, bool b_kmajor, hipStream_t stream);
bool gemm_wave128_f8_mixed_ok(const GemmArgs& p, bool b_kmajor, int rows256);
int gemm_wave128_f8_mixed_launch(const GemmArgs& p, int rows256, bool e5m2, hipStream_t stream);
bool gemm_wave128_f8_192_ok(const GemmArgs& p, bool b_kmajor, int tile_m = 192);   // tiles of 192 x 256 / 128 x 256
bool gemm_wave128_mx_mixed_ok(const GemmArgs& p, int group_bytes, int rows256);
int gemm_wave128_mx_mixed_launch(const GemmArgs& p, int fmt, int rows256, hipStream_t stream);   // fmt: 0 = MXFP4, else MXFP8
bool gemm_wave128_mx_192_ok(const GemmArgs& p, int group_bytes, int tile_m = 192);   // in_dtype: C ABI code of the operands' type
int gemm_wave128_launch(const GemmArgs& p, bool bf16, bool b_kmajor, hipStream_t stream);
int gemm_wave128_f8_launch(const GemmArgs& p, bool e5m2, bool b_kmajor, hipStream_t stream);
bool gemm_wave128_mxfp4_ok(const GemmArgs& p);
int gemm_wave128_mxfp4_launch(const GemmArgs& p, hipStream_t stream);
bool gemm_wave128_mxfp8_ok(const GemmArgs& p);
int gemm_wave128_mxfp8_launch(const GemmArgs& p, hipStream_t stream);
bool gemm8_skinny_ok(const GemmArgs& p);  // M <= 32, K a multiple of 256
int gemm8_skinny_launch(const GemmArgs& p, bool e5m2, hipStream_t stream);
bool gemm_skinny_ok(const SkinnyArgs& p, bool y_kmajor, bool x_kmajor, int elem_bytes);
int gemm_skinny_launch(const SkinnyArgs& p, int kind, bool y_kmajor, bool x_kmajor, hipStream_t stream);
int gemm_strided_launch(const GemmStridedArgs& p, hipStream_t stream);   // fp32 FMAs, one thread per 4 x 4 outputs (a second implementation for tests)
int gemm_masked_launch(const GemmStridedArgs& p, hipStream_t stream);    // 64 x 64 tiles on MFMAs with masked loads: any strides and sizes
int mx_gemm_launch(const GemmArgs& p, int fmt, int tile, hipStream_t stream);
int attn_fwd_launch(const AttnArgs& p, bool bf16, hipStream_t stream);
bool attn_fwd_pipe_ok(const AttnArgs& p);
int attn_fwd_pipe_launch(const AttnArgs& p, bool bf16, hipStream_t stream);
int attn_fwd8_launch(const AttnArgs& p, bool e5m2, hipStream_t stream);  // fp8 inputs, V with N contiguous
int attn_bwd_pre_launch(const AttnArgs& p, bool bf16, hipStream_t stream);
int attn_bwd_launch(const AttnArgs& p, bool bf16, hipStream_t stream);
int gemm_rowfused_launch(const RowFusedArgs& p, bool bf16, hipStream_t stream);
int softmax_rows_launch(void* C, int M, int N, int64_t scm, int64_t scn, int dtype, hipStream_t stream);
int clock_probe_launch(unsigned long long* out, unsigned long long real_ticks, hipStream_t stream);
int mfma_burn_launch(float* sink, int shape, int random_operands, int iters, int waves_per_simd, int cus, hipStream_t stream);
int dequant_launch(const uint8_t* codes, float* out, int64_t n, int fmt, hipStream_t stream);

}  // namespace mi355

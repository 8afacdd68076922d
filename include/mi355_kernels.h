/*
 * C ABI of the MI355X (gfx950) tiled-kernel library: dense GEMM (fp16 / bf16 / fp8),
 * block-scaled MX GEMM (MXFP4 / MXFP8), and fused flash-attention forward / backward.
 *
 * Conventions shared by every entry point
 *   - all pointers are DEVICE pointers unless stated otherwise; the caller owns every buffer
 *     (the library allocates nothing and keeps nothing between calls);
 *   - strides are in ELEMENTS of the tensor's dtype (packed fp4: in bytes);
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream); calls are
 *     asynchronous on that stream and never synchronise;
 *   - the return value is 0 on success, a positive hipError_t when a launch failed, or a
 *     negative MI355_E* code when an argument was rejected before anything was launched.
 *     Nothing is thrown across this boundary.
 *
 * The reference interfaces each entry point stands in for are cited per function as
 * path:line relative to the openai/triton source tree.
 */
#ifndef MI355_KERNELS_H
#define MI355_KERNELS_H

#include <stdint.h>
#include <stddef.h>

/* Version of this interface, returned by mi355_query(MI355_Q_ABI_VERSION).  It goes up whenever an entry point, an
 * enum value or the meaning of an argument is added; a binding built for version V works with any library that
 * reports at least V.  (1: GEMM, MX GEMM, attention, dequant; 2: stream-K with and without a workspace, chained
 * product, clock probe, environment refresh, MI355_ESCRATCH, head dims 16 / 32 / 256 in the backward, fp8 output
 * of the MFMA epilogues; 3: MFMA burn probe with its block-scaled shapes, per-device properties, fp8 attention forward at
 * head dims 16 / 32 / 256, a row-major fp8 B on the MFMA kernels, block-scaled products with any K that is a multiple of
 * 32 and scale rows of any pitch on the MFMA kernels; 4: mi355_gemm_splitk, a row-major B whose N is not a multiple of
 * 16 bytes inside a padded pitch on the tile kernels; 5: fp32 operands in mi355_gemm.) */
#define MI355_ABI_VERSION 5

#ifdef __cplusplus
extern "C" {
#endif

/* element types (the reference's names: python/triton/language/core.py:324-381) */
enum {
  MI355_F16 = 0,    /* fp16                        */
  MI355_BF16 = 1,   /* bf16                        */
  MI355_F8E4M3 = 2, /* fp8e4nv  (OCP e4m3fn)       */
  MI355_F8E5M2 = 3, /* fp8e5    (OCP e5m2)         */
  MI355_F32 = 4     /* fp32 (outputs; operands of mi355_gemm / _tuned / _epilogue) */
};

/* MX element formats for mi355_mx_gemm */
enum {
  MI355_MXFP4 = 0, /* e2m1, two codes per byte, element 2i in the low nibble */
  MI355_MXFP8 = 1  /* e4m3fn, one code per byte                              */
};

/* code formats for mi355_dequant */
enum {
  MI355_DEQ_E4M3 = 0, /* one e4m3fn code per byte                          */
  MI355_DEQ_E5M2 = 1, /* one e5m2 code per byte                            */
  MI355_DEQ_E2M1 = 2, /* two e2m1 codes per byte, low nibble first         */
  MI355_DEQ_E8M0 = 3  /* one e8m0 scale per byte: 2^(b-127), 255 -> NaN    */
};

/* activation fused on the fp32 accumulator (python/tutorials/03-matrix-multiplication.py:304-307, 320-322) */
enum { MI355_ACT_NONE = 0, MI355_ACT_LEAKY_RELU = 1 };

/* argument-error codes (negative); positive return values are hipError_t */
enum {
  MI355_OK = 0,
  MI355_EINVAL = -1,   /* null pointer, non-positive size, unknown enum           */
  MI355_EDTYPE = -2,   /* dtype combination not supported                         */
  MI355_ESHAPE = -3,   /* shape constraint of the kernel family violated          */
  MI355_ESTRIDE = -4,  /* stride / alignment constraint violated                  */
  MI355_EDEVICE = -5,  /* no gfx950 device current                                */
  MI355_ESCRATCH = -6  /* the call needs more than the library's static scratch   */
};

/* mi355_query selectors */
enum {
  MI355_Q_ABI_VERSION = 0,
  MI355_Q_CU_COUNT = 1,
  MI355_Q_IS_GFX950 = 2,
  MI355_Q_LDS_BYTES = 3,
  MI355_Q_CLOCK_KHZ = 4,
  MI355_Q_STREAMK_WORKSPACE_BYTES = 5, /* workspace mi355_gemm_streamk needs on this device */
  MI355_Q_WALL_CLOCK_KHZ = 6           /* rate of the constant real-time counter (mi355_clock_probe) */
};

/*
 * C[M,N] = act( (a_scale*b_scale) * A[M,K] @ B[K,N] ), fp32 accumulation, one rounding to out_dtype.
 *
 * Stands in for the launch of `matmul_kernel` by the host wrappers
 *   python/tutorials/03-matrix-multiplication.py:241-316 (kernel), :330-348 (`matmul`)
 *   python/tutorials/09-persistent-matmul.py:48-102 (kernel), :105-138 (`matmul`, fp8e4nv)
 * i.e. what the generated launcher third_party/amd/backend/driver.py:326-377 does for them.
 * Same arguments as the kernel: three pointers, M N K, six strides (any strides are accepted;
 * the tiled MFMA kernels need a unit stride on one axis of each operand and rows that start on 16-byte boundaries -
 * either layout of B for every type; K a multiple of 16 bytes, N any size when a row-major B's pitch covers N rounded up
 * to 16 bytes -, anything else runs a slower MFMA kernel of 64x64 tiles with masked element loads), plus ACTIVATION.  in_dtype is the type of A and B
 * (they must match, python/triton/language/semantic.py:1355): fp16, bf16, fp8e4nv, fp8e5 or fp32.  fp32 operands are
 * multiplied exactly on the fp32 MFMAs (the `ieee` input precision of `tl.dot`, semantic.py:1322-1410; what the
 * reference's CPU path computes, python/triton/runtime/interpreter.py:542-549) when A's rows and B's columns are
 * K-contiguous and start on 16-byte boundaries with K a multiple of 4, and by an fp32 FMA kernel otherwise.  a_scale / b_scale are
 * optional device pointers to one fp32 each (NULL = 1.0): per-tensor dequantisation
 * scales for fp8 inputs, applied to the fp32 accumulator before activation and cast.
 */
int mi355_gemm(const void* A, const void* B, void* C,
               int M, int N, int K,
               int64_t stride_am, int64_t stride_ak,
               int64_t stride_bk, int64_t stride_bn,
               int64_t stride_cm, int64_t stride_cn,
               int in_dtype, int out_dtype,
               const float* a_scale, const float* b_scale,
               int activation, void* stream);

/* mi355_gemm with the kernel configuration chosen by the caller instead of the library's size
 * heuristic: what the reference's autotuner does when it launches its best `Config`
 * (python/triton/runtime/autotuner.py:146-179 `Autotuner.run`; the configs of the matmul
 * tutorial, python/tutorials/03-matrix-multiplication.py:168-239, differ in tile shape,
 * GROUP_SIZE_M, stages and warps).  tile: -1 = heuristic, 0 = 256x256 ping-pong, 1 = 128x128,
 * 2 = 256x256 one barrier per K step, 3 / 4 = 256x256 software-pipelined with four / eight waves,
 * 5 = the eight-wave pipelined kernel as persistent programs (one per CU, MI355_GEMM_PROGRAMS
 * overrides) that walk their tiles as one stream of K steps, the schedule of
 * python/tutorials/09-persistent-matmul.py:141-190, 6 = four waves of 128x128 from 16x16x32
 * (fp8: 16x16x128) MFMAs on 256x256 tiles (whole tiles, K at least 128 elements - fp8: at least 256 bytes, any multiple of 16 with a
 * K-major B, a multiple of 256 with a row-major one -, a row-major 16-bit B with a pitch that is a multiple of 512 bytes; the
 * heuristic's choice for such products from
 * 128 tiles on, fp8 from 192; with more tiles than MI355_GEMM_PROGRAMS, default the CU count, its programs
 * take ceil(tiles / programs) tiles each as one stream of K steps)
 * (a kernel that does not exist for the dtype or shape falls back to the nearest one).  group_m: the
 * reference's GROUP_SIZE_M (:265-273), 0 = default 8.  Operands without 16-byte rows run the
 * masked any-stride kernel whatever `tile` says.
 */
int mi355_gemm_tuned(const void* A, const void* B, void* C,
                     int M, int N, int K,
                     int64_t stride_am, int64_t stride_ak,
                     int64_t stride_bk, int64_t stride_bn,
                     int64_t stride_cm, int64_t stride_cn,
                     int in_dtype, int out_dtype,
                     const float* a_scale, const float* b_scale,
                     int activation, int tile, int group_m, void* stream);

/* mi355_gemm with K split over `splits` workgroups per tile (0 = chosen by size: one workgroup per CU, at least sixteen
 * 64-byte K steps each, at most 32; none from half a round of 128x128 tiles on): for products of few tiles with a long K - one row of tiles against a long
 * weight, a small square against a long K -, where one workgroup per tile leaves most of the device idle and a few
 * K steps of loads in flight are all that hides the memory latency.  The reference's kernel has no such form
 * (python/tutorials/03-matrix-multiplication.py:241-316 gives every tile to one program); the contract is the same
 * C = act((a_scale * b_scale) * A @ B) with fp32 accumulation and one rounding, the partial sums added in split order.
 * Two launches: the tile kernel on 128x128 tiles into fp32 slices of `workspace`, then the sum and the epilogue.
 * workspace: device memory of at least splits * M * N * 4 bytes (32 * M * N * 4 always suffices for splits = 0),
 * 16-byte aligned, contents irrelevant; two calls that overlap in time need different workspaces.  fp32 operands (K-major B)
 * are split too, and sooner: their products are bound by the fp32 MFMA rate alone, so idle CUs are all that counts.  Operands that the
 * tile kernels do not take, or a K too short to split, run as mi355_gemm (the workspace is then not touched).
 */
int mi355_gemm_splitk(const void* A, const void* B, void* C,
                      int M, int N, int K,
                      int64_t stride_am, int64_t stride_ak,
                      int64_t stride_bk, int64_t stride_bn,
                      int64_t stride_cm, int64_t stride_cn,
                      int in_dtype, int out_dtype,
                      const float* a_scale, const float* b_scale,
                      int activation, int splits, void* workspace, size_t workspace_bytes, void* stream);

/* mi355_gemm with a stream-K schedule: one program per CU, and the programs split ALL K steps of ALL
 * 256x256 tiles evenly, so a tile count that is not a multiple of the CU count (or smaller than it:
 * then this is split-K) still keeps every CU busy to the end.  The persistent schedule of
 * python/tutorials/09-persistent-matmul.py:141-190 deals whole tiles; this deals their K steps.
 * A program that covers only part of a tile leaves fp32 partial sums in `workspace` (caller-owned,
 * at least mi355_query(MI355_Q_STREAMK_WORKSPACE_BYTES) bytes, 16-byte aligned, contents
 * irrelevant before and after the call) and a second launch on the same stream adds the parts up
 * in a fixed order: results do not depend on timing.  Nothing waits for another program, so
 * the call is safe next to other work on the device.  Takes effect for fp16 / bf16 / fp8 operands on
 * the MFMA path with M and N multiples of 256 and K a multiple of 128 elements (256 for fp8);
 * any other call runs exactly as mi355_gemm.
 */
int mi355_gemm_streamk(const void* A, const void* B, void* C,
                       int M, int N, int K,
                       int64_t stride_am, int64_t stride_ak,
                       int64_t stride_bk, int64_t stride_bn,
                       int64_t stride_cm, int64_t stride_cn,
                       int in_dtype, int out_dtype,
                       const float* a_scale, const float* b_scale,
                       int activation, void* workspace, size_t workspace_bytes, void* stream);

/* mi355_gemm_streamk for callers that cannot allocate (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc): the same kernels, with the partial-tile workspace in a static device
 * array of the library instead of a caller's buffer.  No counterpart in the reference.  The call performs
 * no hipMalloc / hipFree and calls no allocating routine.  Limit: the array is 128 MiB per GPU (two
 * 256x256 fp32 tiles for each of at most 256 programs, one program per compute unit; every GPU the library
 * runs on holds it until the process ends); a device or MI355_GEMM_PROGRAMS setting that would need more
 * programs returns MI355_ESCRATCH.  The first call on a device looks the array's address up (do it once
 * before capturing a graph).  All calls on one GPU share that GPU's array: two calls that overlap in time
 * on one GPU (different streams, or threads) race and give wrong results - serialise them.  Its contents are
 * irrelevant before and after a call (every slot a call reads, the same call wrote), so nothing is cleared.
 */
int mi355_gemm_streamk_static(const void* A, const void* B, void* C,
                              int M, int N, int K,
                              int64_t stride_am, int64_t stride_ak,
                              int64_t stride_bk, int64_t stride_bn,
                              int64_t stride_cm, int64_t stride_cn,
                              int in_dtype, int out_dtype,
                              const float* a_scale, const float* b_scale,
                              int activation, void* stream);

/* mi355_gemm with the epilogues of the reference's dot test fused in:
 *   C = softmax_rows?( act( (a_scale * b_scale) * A @ B + D ) )
 *
 * Stands in for the ADD_MATRIX / ADD_ROWS / ADD_COLS / DO_SOFTMAX branches of the kernel in
 *   python/test/unit/language/test_core.py:3128-3141 (and its checks, :3226-3235)
 * and keeps the ACTIVATION hook of python/tutorials/03-matrix-multiplication.py:304-307.
 * D ("addend", NULL = none) is read as D[m * stride_dm + n * stride_dn]; a zero stride
 * broadcasts: stride_dn = 0 is the reference's add-rows (one value per row of C), stride_dm = 0
 * its add-cols (one value per column), both non-zero its add-matrix.  D is fp16, bf16 or fp32
 * (addend_dtype) and is added to the fp32 accumulator before the activation and the one
 * rounding to out_dtype.  The add-matrix form may alias C (the reference adds the previous
 * contents of Z); a broadcast D must not overlap C.
 * softmax = 1 then replaces every row of C by exp(c - max) / sum (fp32 arithmetic).  With fp16 / bf16
 * operands and N <= 256 - a row fits one tile, the reference's case - product, addend, activation and
 * softmax are ONE launch on the fp32 accumulator with one rounding at the store; wider rows are
 * normalised by a second launch on the same stream, which re-reads the rounded C.
 * CHAIN_DOT (:3142-3144) is mi355_gemm_chain below.
 */
int mi355_gemm_epilogue(const void* A, const void* B, void* C,
                        int M, int N, int K,
                        int64_t stride_am, int64_t stride_ak,
                        int64_t stride_bk, int64_t stride_bn,
                        int64_t stride_cm, int64_t stride_cn,
                        int in_dtype, int out_dtype,
                        const float* a_scale, const float* b_scale,
                        const void* addend, int64_t stride_dm, int64_t stride_dn, int addend_dtype,
                        int activation, int softmax, void* stream);

/*
 * C[M,N2] = z^ @ W with z = softmax_rows?( act( (a_scale * b_scale) * A[M,K] @ B[K,N] + D ) ) and z^ = z rounded
 * to the operand type: the CHAIN_DOT branch of the reference's dot test,
 *   python/test/unit/language/test_core.py:3142-3144  `z = tl.dot(z.to(w.dtype), w)`
 * (with the branches before it, :3128-3141, as in mi355_gemm_epilogue), in ONE launch: z stays in registers
 * between the two products, as it stays inside the reference's single tile; fp32 accumulation in both, one
 * rounding to out_dtype at the store (:3145).  A, B, W are fp16 or bf16 (in_dtype) with any element strides;
 * the intermediate row must fit one tile: N <= 256 and N2 <= 256, else MI355_ESHAPE (chain two mi355_gemm calls).
 */
int mi355_gemm_chain(const void* A, const void* B, const void* W, void* C,
                     int M, int N, int K, int N2,
                     int64_t stride_am, int64_t stride_ak,
                     int64_t stride_bk, int64_t stride_bn,
                     int64_t stride_wn, int64_t stride_wn2,
                     int64_t stride_cm, int64_t stride_cn,
                     int in_dtype, int out_dtype,
                     const float* a_scale, const float* b_scale,
                     const void* addend, int64_t stride_dm, int64_t stride_dn, int addend_dtype,
                     int activation, int softmax, void* stream);

/*
 * Grouped GEMM: C_g[M_g,N_g] = A_g[M_g,K_g] @ B_g[K_g,N_g] for g = 0 .. group_size-1 in ONE launch.
 *
 * Stands in for the launch of `grouped_matmul_kernel` by `group_gemm_fn`
 *   python/tutorials/08-grouped-gemm.py:64-140 (kernel), :143-187 (host wrapper)
 * with the kernel's own arguments: device arrays of matrix addresses (uint64), a device int32 array
 * `d_sizes[group_size][3]` = <M, N, K> and a device int32 array `d_lds[group_size][3]` =
 * <lda, ldb, ldc> in elements; all matrices row major (unit column stride), A, B and C of type
 * `dtype` (MI355_F16 as in the reference, or MI355_BF16), fp32 accumulation.
 * `num_programs` workgroups walk the tiles of all problems (the reference's NUM_SM); 0 picks two
 * per compute unit.  Any sizes are accepted (partial tiles are handled; the reference assumes
 * full tiles); problems whose lda, ldb, N or K are not multiples of 8 elements, or whose A / B
 * are not 16-byte aligned, run a slower loop inside the same kernel.  Groups in which every problem
 * is whole 256x256 tiles with K a multiple of 128 (and ldb a multiple of 256 elements) run a faster
 * kernel from one tile per compute unit and K >= 512 on.  Nothing about the device
 * arrays can be checked on the host: they must hold `group_size` valid entries.
 */
int mi355_grouped_gemm(const void* d_a_ptrs, const void* d_b_ptrs, const void* d_c_ptrs,
                       const int32_t* d_sizes, const int32_t* d_lds, int group_size,
                       int dtype, int num_programs, void* stream);

/*
 * Block-scaled (OCP MX v1.0) GEMM: C[m,n] = sum_kb 2^(sA[m,kb]-127) 2^(sB[n,kb]-127) sum_{k in kb} A^[m,k] B^[n,k]
 * with 32-element blocks along K.  A is [M, K] and B is [N, K] (both K-contiguous):
 *   MXFP4: A_bytes[M, K/2], B_bytes[N, K/2];   MXFP8: A_bytes[M, K], B_bytes[N, K];
 *   scales: sA[M, K/32], sB[N, K/32] e8m0 bytes (2^(b-127)); C[M,N] in out_dtype (bf16/fp16/fp32).
 * lda/ldb are row pitches in BYTES, lds_a/lds_b row pitches of the scale matrices in bytes, ldc in elements.
 * No counterpart exists in the reference snapshot (no dot_scaled / e8m0 / e2m1 anywhere in it);
 * the operation is defined by the OCP Microscaling Formats specification v1.0.
 */
int mi355_mx_gemm(const uint8_t* A, const uint8_t* sA, const uint8_t* B, const uint8_t* sB, void* C,
                  int M, int N, int K, int fmt, int out_dtype,
                  int64_t lda, int64_t ldb, int64_t lds_a, int64_t lds_b, int64_t ldc,
                  void* stream);

/*
 * Flash-attention forward: O = softmax(Q K^T * sm_scale [+ causal mask]) V per (z, h); also writes
 * Mlse[z,h,n] = base-2 log-sum-exp of (q.k * sm_scale * log2 e), fp32.
 * Stands in for the launch of `_attn_fwd` by `_attention.forward`
 *   python/tutorials/06-fused-attention.py:98-187 (kernel), :25-75 (inner loop), :441-475 (host).
 * q,k,v,o are [Z,H,N_CTX,D] with the four element strides given per tensor (last stride must be 1);
 * Mlse is contiguous [Z,H,N_CTX].  dtype is MI355_F16 or MI355_BF16; D in {16, 32, 64, 128, 256}
 * (forward and backward entries alike; 16 and 32, the reference's other two head dims, :447, are taken as they
 * are - rows of D elements - and run the 64-column kernels in a form that pads with zeros on the fly).
 * fp8 forward (dtype MI355_F8E5M2 as in the reference's fp8 benchmark, :609-614, or MI355_F8E4M3):
 * q, k and o as above, v transposed in memory (stride 1 along N_CTX, a multiple of 16 along D:
 * what `v.permute(0,1,3,2).contiguous().permute(0,1,3,2)` yields); P is rounded to the fp8 type
 * before the second product (:66-67) and o is written in the fp8 type; the same five head dims (16 and 32: rows
 * of D bytes, and D rows of V^T).  There is no fp8 backward.
 */
int mi355_attn_fwd(const void* q, const void* k, const void* v, void* o, float* Mlse,
                   int Z, int H, int N_CTX, int D,
                   const int64_t* stride_q, const int64_t* stride_k,
                   const int64_t* stride_v, const int64_t* stride_o, /* HOST arrays of 4 */
                   float sm_scale, int causal, int dtype, void* stream);

/*
 * delta[z,h,n] = sum_d o[z,h,n,d] * do[z,h,n,d] in fp32.
 * Stands in for `_attn_bwd_preprocess` (python/tutorials/06-fused-attention.py:190-204, launch :495-502).
 * o and do share `stride` (HOST array of 4, last = 1); delta is contiguous [Z,H,N_CTX].
 */
int mi355_attn_bwd_preprocess(const void* o, const void* d_o, float* delta,
                              int Z, int H, int N_CTX, int D,
                              const int64_t* stride, int dtype, void* stream);

/*
 * Flash-attention backward: dq, dk, dv from q, k, v, do, Mlse (from the forward) and delta.
 * Stands in for the launch of `_attn_bwd` by `_attention.backward`
 *   python/tutorials/06-fused-attention.py:308-435 (kernel), :208-305 (inner loops), :478-517 (host).
 * All of q,k,v,do,dq,dk,dv share one stride set (HOST array of 4, last = 1), as in the reference (:481):
 * only that one array is passed and validated, every tensor is addressed with it and must be 16-byte aligned;
 * a caller whose tensors differ in strides must make them alike first (the reference asserts it, :481).
 * k is the ORIGINAL key tensor: the pre-scaling `k * (sm_scale / ln 2)` the reference does on the
 * host (:490-492) is folded into the kernel.  causal = 0 gives the full (non-causal) backward,
 * which the reference kernel cannot produce.  N_CTX must be a multiple of 128 (:494).
 */
int mi355_attn_bwd(const void* q, const void* k, const void* v, const void* d_o,
                   const float* Mlse, const float* delta,
                   void* dq, void* dk, void* dv,
                   int Z, int H, int N_CTX, int D,
                   const int64_t* stride,
                   float sm_scale, int causal, int dtype, void* stream);

/*
 * out[i] = decode(codes[i]) in fp32 for n code BYTES (MI355_DEQ_E2M1 writes 2n values), using the
 * decode routines the strided kernels use.  The formats are those of the reference type table
 * (python/triton/language/core.py:352-363) and of its up-cast emulation
 * (python/triton/runtime/interpreter.py:130-191, python/test/unit/language/test_conversions.py:178-209);
 * e2m1 / e8m0 follow OCP MX v1.0.
 */
int mi355_dequant(const uint8_t* codes, float* out, int64_t n, int fmt, void* stream);

/*
 * Shader clock under load: a one-wave kernel that lives for `duration_us` (at most 2 s) of real time on
 * `stream` and then writes ticks[0] = shader-clock cycles and ticks[1] = real-time counter ticks that
 * passed (device memory, two uint64, 8-byte aligned).  Launched on a second stream next to the kernels
 * under study, clock = ticks[0] / ticks[1] * mi355_query(MI355_Q_WALL_CLOCK_KHZ) is the clock they ran at:
 * the board lowers the clock of MFMA-heavy kernels to hold its power limit, so peak fractions computed
 * from the nominal clock (as python/triton/testing.py:404-426 `get_max_tensorcore_tflops` does from a
 * clock argument) need the observed one.  Asynchronous like every other entry.
 */
int mi355_clock_probe(uint64_t* ticks, int duration_us, void* stream);

/*
 * What the matrix pipes of this board sustain: every SIMD of every CU runs `waves_per_simd` (1 or 2) waves that issue
 * `iters` rounds of one MFMA shape back to back from registers - no memory traffic -, on pseudo-random operand bits
 * (`random_operands` != 0: finite values, the switching activity of real data) or on one constant.  One round is
 * 8 x 32768 flop per wave for the 16-bit shapes, twice that for fp8, four times for fp4, so a launch is
 * CUs x 4 x waves_per_simd x iters x 262144 x {1, 2, 4} flop; the caller times it with events and reads watts and
 * clock next to it.  Under the board's power limit this, not the nominal peak, is what a GEMM built from that MFMA
 * shape can approach.  `sink` is one float of device memory (practically never written).  The measurement analogue of
 * the reference's peak helper (python/triton/testing.py:404-426), which takes its rate from a table.
 */
enum {
  MI355_BURN_BF16_32X32X16 = 0,
  MI355_BURN_BF16_16X16X32 = 1,
  MI355_BURN_FP8_32X32X64 = 2,
  MI355_BURN_FP8_16X16X128 = 3,
  MI355_BURN_FP4_32X32X64 = 4,
  MI355_BURN_FP4_16X16X128 = 5,
  MI355_BURN_MXFP4_32X32X64 = 6,    /* the block-scaled forms of the two fp4 shapes (one e8m0 scale per lane and operand) */
  MI355_BURN_MXFP4_16X16X128 = 7
};
int mi355_mfma_burn(float* sink, int shape, int random_operands, int iters, int waves_per_simd, void* stream);

/* Device facts needed by callers (analogue of get_device_properties,
 * third_party/amd/backend/driver.c:125-141).  Returns -1 for an unknown selector. */
int mi355_query(int what);

/* The library reads its MI355_* tuning variables from the environment once, at the first call that
 * needs one (the reference reads its own per call or per import: python/triton/runtime/jit.py:717,
 * :848, python/triton/runtime/autotuner.py:166); this reads them again, for a caller that changed
 * them afterwards.  Not to be called while another thread is inside the library. */
void mi355_refresh_env(void);

/* Static string for a return code of the functions above (never NULL). */
const char* mi355_strerror(int code);

#ifdef __cplusplus
}
#endif
#endif /* MI355_KERNELS_H */

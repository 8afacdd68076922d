// extern "C" entry points declared in include/mi355_kernels.h: argument validation, kernel
// family / tile selection, launch.  Plays the role of the generated launcher of the reference
// (third_party/amd/backend/driver.py:326-377): pointers and scalars in, one asynchronous
// launch on the caller's stream out, an integer status back.
#include <algorithm>
#include <cmath>
#include <hip/hip_runtime.h>
#include <stdlib.h>
#include <string.h>
#include <atomic>
#include <climits>
#include <mutex>
#include "../../include/mi355_kernels.h"
#include "launch.h"

using namespace mi355;

namespace {

struct DeviceInfo {
  int ok = 0, cus = 0, gfx950 = 0, lds = 0, clock_khz = 0, wall_clock_khz = 0;
};

// properties of the CURRENT device, read once per device (a process may hold several)
const DeviceInfo& device_info() {
  constexpr int kMax = 64;
  static DeviceInfo infos[kMax];
  static std::atomic<int> ready[kMax];
  static std::mutex mutex;
  static const DeviceInfo none;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMax) return none;
  if (ready[dev].load(std::memory_order_acquire)) return infos[dev];
  std::lock_guard<std::mutex> lock(mutex);
  if (ready[dev].load(std::memory_order_relaxed)) return infos[dev];
  DeviceInfo& info = infos[dev];
  hipDeviceProp_t prop;
  if (hipGetDeviceProperties(&prop, dev) != hipSuccess) return none;
  info.cus = prop.multiProcessorCount;
  info.gfx950 = strncmp(prop.gcnArchName, "gfx950", 6) == 0;
  info.lds = (int)prop.sharedMemPerBlock;
  info.clock_khz = prop.clockRate;
  if (hipDeviceGetAttribute(&info.wall_clock_khz, hipDeviceAttributeWallClockRate, dev) != hipSuccess) info.wall_clock_khz = 0;
  info.ok = 1;
  ready[dev].store(1, std::memory_order_release);
  return info;
}

// Tuning knobs from the environment (the reference's third configuration mechanism: environment
// variables read by the runtime, python/triton/runtime/jit.py:717, :848).  Read ONCE per process, at the
// first call that needs them, and again only when mi355_refresh_env() is called: a launch costs no getenv.
// UNSET = the variable is absent or empty and the call site's own default applies.
constexpr int UNSET = INT_MIN;
struct Knobs {
  int force_strided, group_m, tile, programs, skinny, grouped_big_min, grouped_wave128_min_k, grouped_chunk,
      attn_fwd_variant, attn_programs, lean_epilogue, tile_m, rowfused_max_mk, mixed_rows;
};
Knobs g_knobs;
std::atomic<int> g_knobs_ready{0};
std::mutex g_knobs_mutex;

int read_env(const char* name, int lo) {
  const char* s = getenv(name);
  if (!s || !*s) return UNSET;
  const int v = atoi(s);
  return v < lo ? lo : v;   // (out-of-range values are clamped, never passed on to a kernel)
}

void load_knobs() {
  std::lock_guard<std::mutex> lock(g_knobs_mutex);
  Knobs k;
  k.force_strided = read_env("MI355_GEMM_FORCE_STRIDED", 0);
  k.group_m = read_env("MI355_GEMM_GROUP_M", 1);
  k.tile = read_env("MI355_GEMM_TILE", -1);   // (-1: the block-scaled products' one-thread-per-output kernel)
  k.programs = read_env("MI355_GEMM_PROGRAMS", 1);
  k.skinny = read_env("MI355_GEMM_SKINNY", 0);
  k.grouped_big_min = read_env("MI355_GROUPED_BIG_MIN", 1);
  k.grouped_wave128_min_k = read_env("MI355_GROUPED_WAVE128_MIN_K", 0);
  k.grouped_chunk = read_env("MI355_GROUPED_CHUNK", 1);
  k.attn_fwd_variant = read_env("MI355_ATTN_FWD_VARIANT", 0);
  k.attn_programs = read_env("MI355_ATTN_PROGRAMS", 1);
  k.lean_epilogue = read_env("MI355_GEMM_LEAN_EPILOGUE", 0);
  k.tile_m = read_env("MI355_GEMM_TILE_M", 0);
  k.rowfused_max_mk = read_env("MI355_ROWFUSED_MAX_MK", 0);
  k.mixed_rows = read_env("MI355_GEMM_MIXED_ROWS", 0);
  g_knobs = k;
  g_knobs_ready.store(1, std::memory_order_release);
}

const Knobs& knobs() {
  if (!g_knobs_ready.load(std::memory_order_acquire)) load_knobs();
  return g_knobs;
}

int knob(int value, int dflt) { return value == UNSET ? dflt : value; }

// Two tile heights in one launch (gemm_wave128_mixed_kernel and its fp8 / block-scaled forms): the rows of C to give to
// the 256-row tiles, the rest going to 192-row tiles, for a product of M rows and nn tile columns on P programs - or 0
// when no split is rated 5 % better than one tile height.  A split is rated by its busiest program (tiles b, b + P, ...
// of the first part and P - 1 - b, ... of the second; a 192-row tile counted as 0.78 of a 256-row one: 3072^3 on 192
// of them against 4096^3 on 256 tiles, per tile and K step); among the splits within 7 % of the best, the one whose two
// parts are closest in work is taken (measured: 5120^3 bf16 1164 / 1280 / 1325 TFLOP/s for 100 + 400 / 160 + 320 / 220 +
// 240 tiles, which the count rates the same).
int mixed_split(int M, int nn, int P) {
  if (M % 256 != 0 || nn <= 0 || P <= 0) return 0;
  auto count = [&](long tiles, int b) { return b < tiles ? (tiles - b + P - 1) / P : 0; };
  const long tiles256 = (long)(M / 256) * nn;
  double one_height = (double)((tiles256 + P - 1) / P), best = 1e30;   // in units of a 256-row tile's time
  if (M % 192 == 0) one_height = std::min(one_height, 0.78 * (double)(((long)(M / 192) * nn + P - 1) / P));
  auto busiest = [&](int a) {
    const long n256 = (long)a * nn, n192 = (long)((M - a * 256) / 192) * nn;
    double worst = 0;
    for (int b = 0; b < P; b++) worst = std::max(worst, (double)count(n256, b) + 0.78 * (double)count(n192, P - 1 - b));
    return worst;
  };
  for (int a = 1; a * 256 < M; a++)
    if ((M - a * 256) % 192 == 0) best = std::min(best, busiest(a));
  if (!(best < 0.95 * one_height)) return 0;
  int best_rows = 0;
  double best_gap = 1e30;
  for (int a = 1; a * 256 < M; a++) {
    if ((M - a * 256) % 192 != 0 || busiest(a) > 1.07 * best) continue;
    const double gap = std::abs((double)a * nn - 0.78 * (double)((M - a * 256) / 192) * nn);
    if (gap < best_gap) { best_gap = gap; best_rows = a * 256; }
  }
  return best_rows;
}

bool aligned(const void* p, size_t a) { return ((uintptr_t)p % a) == 0; }

int elem_size(int dtype) {
  switch (dtype) {
    case MI355_F16: case MI355_BF16: return 2;
    case MI355_F8E4M3: case MI355_F8E5M2: return 1;
    case MI355_F32: return 4;
    default: return 0;
  }
}

bool copy_strides(const int64_t* src, int64_t* dst) {
  if (!src) return false;
  for (int i = 0; i < 4; i++) dst[i] = src[i];
  return true;
}

}  // namespace

extern "C" {

int mi355_query(int what) {
  if (what == MI355_Q_ABI_VERSION) return MI355_ABI_VERSION;   // (answered without touching the device)
  const DeviceInfo& d = device_info();
  switch (what) {
    case MI355_Q_ABI_VERSION: return MI355_ABI_VERSION;
    case MI355_Q_CU_COUNT: return d.cus;
    case MI355_Q_IS_GFX950: return d.gfx950;
    case MI355_Q_LDS_BYTES: return d.lds;
    case MI355_Q_CLOCK_KHZ: return d.clock_khz;
    case MI355_Q_WALL_CLOCK_KHZ: return d.wall_clock_khz;
    case MI355_Q_STREAMK_WORKSPACE_BYTES: return (d.cus > 0 ? d.cus : 256) * 2 * 256 * 256 * 4;
    default: return -1;
  }
}

void mi355_refresh_env(void) { load_knobs(); }

const char* mi355_strerror(int code) {
  switch (code) {
    case MI355_OK: return "ok";
    case MI355_EINVAL: return "invalid argument (null pointer, non-positive size or unknown enum)";
    case MI355_EDTYPE: return "unsupported dtype combination";
    case MI355_ESHAPE: return "shape not supported by this kernel family";
    case MI355_ESTRIDE: return "stride or alignment not supported by this kernel family";
    case MI355_EDEVICE: return "current device is not a gfx950 GPU";
    case MI355_ESCRATCH: return "the library's static scratch array is too small for this call (more than 256 programs)";
    default: break;
  }
  if (code > 0) return hipGetErrorString((hipError_t)code);
  return "unknown error";
}

static int gemm_impl(const void* A, const void* B, void* C, int M, int N, int K,
                     int64_t sam, int64_t sak, int64_t sbk, int64_t sbn, int64_t scm, int64_t scn,
                     int in_dtype, int out_dtype, const float* a_scale, const float* b_scale,
                     int activation, const void* aux, int64_t aux_sm, int64_t aux_sn, int aux_dtype,
                     int tile_arg, int group_m_arg, void* stream_, float* workspace = nullptr) {
  if (!A || !B || !C || M <= 0 || N <= 0 || K <= 0) return MI355_EINVAL;
  if (aux && aux_dtype != MI355_F16 && aux_dtype != MI355_BF16 && aux_dtype != MI355_F32) return MI355_EDTYPE;
  if (activation != MI355_ACT_NONE && activation != MI355_ACT_LEAKY_RELU) return MI355_EINVAL;
  if (in_dtype < MI355_F16 || in_dtype > MI355_F32) return MI355_EDTYPE;
  if (out_dtype < MI355_F16 || out_dtype > MI355_F32) return MI355_EDTYPE;
  if (!device_info().gfx950) return MI355_EDEVICE;
  hipStream_t stream = (hipStream_t)stream_;
  const int es = elem_size(in_dtype);
  const bool is32 = in_dtype == MI355_F32;   // fp32 operands: fp32 MFMAs with a K-major B, the any-stride FMA kernel otherwise
  const bool is8 = es == 1;
  const int vec = 16 / es;  // elements per 16-byte chunk

  const bool out_ok = true;   // every output type of the ABI has a store in the MFMA epilogues (fp8: hardware conversion, saturating)
  const bool a_ok = sak == 1 && sam % vec == 0 && sam >= K && aligned(A, 16) && K % vec == 0;
  const bool b_kmajor = sbk == 1 && sbn % vec == 0 && sbn >= K && aligned(B, 16);
  // (a row-major B: rows of whole 16-byte chunks - N itself need not be one: the last chunk of a row then reaches into
  // the padding that the pitch provides, and the columns beyond N are never stored)
  const bool b_nmajor = !is32 && sbn == 1 && sbk % vec == 0 && sbk >= (N + vec - 1) / vec * vec && aligned(B, 16);
  // the tile copies address 256 rows of an operand with 32-bit byte offsets from a 64-bit tile base
  const bool pitch_ok = (int64_t)sam * es < (1 << 23) && (b_kmajor ? (int64_t)sbn * es < (1 << 23) : (int64_t)sbk * es < (1 << 26));
  const bool fast = pitch_ok && out_ok && a_ok && (b_kmajor || b_nmajor) && knob(knobs().force_strided, 0) == 0;

  if (!fast && is32) {
    GemmStridedArgs s{A, B, C, M, N, K, sam, sak, sbk, sbn, scm, scn, a_scale, b_scale, activation, in_dtype, out_dtype,
                      aux, aux_sm, aux_sn, aux_dtype};
    return gemm_strided_launch(s, stream);   // (the masked MFMA kernel converts to 16 bits on its way through LDS: not for fp32)
  }
  if (!fast) {
    GemmStridedArgs s{A, B, C, M, N, K, sam, sak, sbk, sbn, scm, scn, a_scale, b_scale, activation, in_dtype, out_dtype,
                      aux, aux_sm, aux_sn, aux_dtype};
    // (MI355_GEMM_FORCE_STRIDED=2: the fp32-FMA kernel, a second implementation kept for tests)
    return knob(knobs().force_strided, 0) == 2 ? gemm_strided_launch(s, stream) : gemm_masked_launch(s, stream);
  }

  GemmArgs p{};
  p.A = (const char*)A; p.B = (const char*)B; p.C = (char*)C;
  p.M = M; p.N = N; p.K = K; p.k_bytes = K * es;
  p.lda = sam * es;
  p.ldb = (b_kmajor ? sbn : sbk) * es;
  p.ldc = scm; p.scn = scn;
  p.a_scale = a_scale; p.b_scale = b_scale;
  p.activation = activation; p.out_dtype = out_dtype;
  p.group_m = group_m_arg > 0 ? group_m_arg : knob(knobs().group_m, 8);
  // four consecutive C elements as one store: rows of 16-bit / fp32 elements 16-byte aligned (for fp8 that
  // makes every group of four 4-byte aligned)
  p.c_vec_ok = scn == 1 && scm % 4 == 0 && aligned(C, 16);
  p.lean_ok = knob(knobs().lean_epilogue, 1);
  p.aux = aux; p.aux_sm = aux_sm; p.aux_sn = aux_sn; p.aux_dtype = aux_dtype;

  const int cus = device_info().cus > 0 ? device_info().cus : 256;
  // 256x256 tiles once they fill half of the CUs, 128x128 tiles (two workgroups per CU) below that
  // (bf16, 144 tiles: 912 vs 651 TFLOP/s; 100 tiles: 654 vs 715)
  const long tiles256 = (long)((M + 255) / 256) * ((N + 255) / 256);
  if (is32) {
    p.num_programs = std::min(knob(knobs().programs, cus), cus);
    // fp32 products are bound by the fp32 MFMA rate alone (1/16 of the bf16 rate on the same bytes), so what counts is
    // how evenly the tiles fill the CUs: 256x256 tiles (pipelined kernel: 8192^3 152 TFLOP/s, 4096^3 149; one barrier per
    // step 141 / 139) against 128x128 tiles, two workgroups per CU, at about 0.9 of that rate (137 / 135; 2048^3: 102
    // against 36 for its 64 large tiles)
    auto fill = [&](long t, long slots) { return (double)t / (double)(((t + slots - 1) / slots) * slots); };
    const long tiles128 = (long)((M + 127) / 128) * ((N + 127) / 128);
    const bool large = fill(tiles256, cus) >= 0.9 * fill(tiles128, 2 * cus);
    const int t32 = tile_arg >= 0 ? tile_arg : knob(knobs().tile, large ? (tiles256 % cus == 0 ? 5 : 4) : 1);
    return gemm32_launch(p, t32 == 6 || t32 == 7 ? 4 : t32, stream);   // (the four-wave 16x16 kernels and stream-K have no fp32 form)
  }
  // large problems run the software-pipelined 8-wave kernel
  // (5 = the persistent form of the pipelined kernel; it falls back to 4 for edge tiles or a K tail)
  // persistent only when every program gets the same number of tiles: with a remainder the hardware's
  // dynamic dispatch of one workgroup per tile balances better (6144^3: 1011 vs 942 TFLOP/s)
  int tile = (tiles256 * 2 >= cus) ? (tiles256 % cus == 0 ? 5 : 4) : 1;
  // 16-bit operands, whole 256x256 tiles and K steps, at least half a round of tiles: four waves of
  // 16x16x32 MFMAs, one workgroup per tile (at 8192^3 bf16 +5 % over the persistent form with a row-major
  // B, +14 % with a K-major B; at 3072^3, 144 tiles, 790 vs 660 TFLOP/s for the 128x128 tiles)
  // (fp8, K-major B: 16x16x128 MFMAs, 8192^3 e4m3 2790-2810 vs 2570-2600 TFLOP/s)
  // (an epilogue addend: instantiations of their own)
  // (fp8 from three quarters of a round: at 144 tiles the eight-wave kernel is 4-7 % ahead - 3072^3 1520 vs
  // 1450, 3072x3072x8192 2040 vs 1890 TFLOP/s -, at 196 tiles the four-wave one by 2 %, at 225 by 13 %)
  const bool w128_ok = is8 ? gemm_wave128_f8_ok(p, b_kmajor) : gemm_wave128_ok(p, b_kmajor, in_dtype);
  if (tiles256 * (is8 ? 4 : 2) >= cus * (is8 ? 3 : 1) && w128_ok) tile = 6;
  tile = tile_arg >= 0 ? tile_arg : knob(knobs().tile, tile);
  // 16-bit products whose 256 x 256 tiles fill the last round of CUs badly (or whose M is a multiple of 192 only): the
  // same kernel on tiles of 192 x 256 where those use the CUs better (3072^3: 192 tiles instead of 144 for 256 CUs)
  if (!is8 && tile_arg < 0 && (knobs().tile == UNSET || knobs().tile_m == 192) && gemm_wave128_192_ok(p, b_kmajor, in_dtype)) {
    auto fill = [&](long t) { return t <= 0 ? 0.0 : (double)t / (double)(((t + cus - 1) / cus) * cus); };
    const long tiles192 = (long)(M / 192) * (N / 256);
    const int want = knob(knobs().tile_m, 0);
    // (below half a round of 256-row tiles the 128-row tiles further down may fill better still: 3072 x 2048 x 4096 bf16,
    // 128 tiles of 192 rows 734 TFLOP/s, 192 tiles of 128 rows 815)
    const long tiles128 = (long)(M / 128) * (N / 256);
    const bool rather128 = tile == 1 && M % 128 == 0 && tiles128 <= cus && fill(tiles128) > fill(tiles192) &&
                           gemm_wave128_192_ok(p, b_kmajor, in_dtype, 128);
    if (want == 192 || (want == 0 && !rather128 && tiles192 * 2 >= cus && (tile != 6 || fill(tiles192) > fill(tiles256) + 0.08))) {
      tile = 6;
      p.tile_m = 192;
    }
  }
  // fp8 likewise (K-major B, 16-bit C), from three quarters of a round of the 192-row tiles on.  Flushed do_bench, e4m3,
  // 256-row choice / 192-row tiles: 3072^3 (144 / 192 tiles) 1100 / 1565 TFLOP/s, 3072 x 3072 x 8192 1365 / 2145, 2304 x
  // 4096 x 4096 1220 / 1785, 4608 x 4096 x 4096 (288 / 384) 1600 / 2070, 6144^3 (576 / 768) 2510 / 2805, 1536 x 8192 x 8192
  // (192 / 256) 2100 / 2680; not taken where they fill worse: 3840 x 3840 x 4096 (225 / 300) 2270 / 1530, 5376 x 5120 x
  // 4096 (420 / 560) 2185 / 1995
  if (is8 && tile_arg < 0 && (knobs().tile == UNSET || knobs().tile_m == 192) && gemm_wave128_f8_192_ok(p, b_kmajor)) {
    auto fill = [&](long t) { return t <= 0 ? 0.0 : (double)t / (double)(((t + cus - 1) / cus) * cus); };
    const long tiles192 = (long)(M / 192) * (N / 256);
    const int want = knob(knobs().tile_m, 0);
    if (want == 192 || (want == 0 && tiles192 * 4 >= cus * 3 && (tile != 6 || fill(tiles192) > fill(tiles256) + 0.08))) {
      tile = 6;
      p.tile_m = 192;
    }
  }
  // and on tiles of 128 x 256 where the 256 x 256 tiles are too few for their kernel (less than half a round) but these
  // fill more than half of one round (2560^3: 100 and 200 tiles; 716 -> 825 TFLOP/s against the 128 x 128 tiles; 2304 x
  // 2048 x 8192, 144 tiles: 650 -> 692; at half a round the 128 x 128 tiles stay ahead, 2048 x 2048 x 4096: 627 vs 569)
  if (!is8 && tile_arg < 0 && (knobs().tile == UNSET || knobs().tile_m == 128) && p.tile_m == 0 &&
      gemm_wave128_192_ok(p, b_kmajor, in_dtype, 128)) {
    const long tiles128 = (long)(M / 128) * (N / 256);
    const int want = knob(knobs().tile_m, 0);
    if (want == 128 || (want == 0 && tile == 1 && tiles128 * 16 >= cus * 9 && tiles128 <= cus)) {
      tile = 6;
      p.tile_m = 128;
    }
  }
  // fp8 likewise (measured: see the design notes' table of shapes)
  if (is8 && tile_arg < 0 && (knobs().tile == UNSET || knobs().tile_m == 128) && p.tile_m == 0 &&
      gemm_wave128_f8_192_ok(p, b_kmajor, 128)) {
    const long tiles128 = (long)(M / 128) * (N / 256);
    const int want = knob(knobs().tile_m, 0);
    if (want == 128 || (want == 0 && tile == 1 && tiles128 * 16 >= cus * 9 && tiles128 <= cus)) {
      tile = 6;
      p.tile_m = 128;
    }
  }
  // 16-bit and fp8 products of more than one round of tiles whose last round is badly filled: the upper rows on 256-row
  // tiles and the lower ones on 192-row tiles in ONE launch, split by mixed_split.  MI355_GEMM_MIXED_ROWS forces the rows
  // of the 256-row part (0 = never).
  int mixed_rows = 0;
  auto mixed_ok = [&](int rows256) {
    return is8 ? gemm_wave128_f8_mixed_ok(p, b_kmajor, rows256) : gemm_wave128_mixed_ok(p, b_kmajor, in_dtype, rows256);
  };
  if (tile_arg < 0 && knobs().tile == UNSET && knobs().tile_m == UNSET && N % 256 == 0) {
    const int want = knob(knobs().mixed_rows, -1);
    const int nn = N / 256, P = cus;
    if (want > 0) {
      if (mixed_ok(want)) mixed_rows = want;
    } else if (want < 0 && tile == 6 && p.tile_m == 0 && tiles256 > cus && M % 256 == 0) {
      const int rows = mixed_split(M, nn, P);
      if (rows > 0 && mixed_ok(rows)) mixed_rows = rows;
    }
  }
  p.num_programs = knob(knobs().programs, cus);  // persistent and stream-K forms (tile 5 / 7): one workgroup per CU
  if (p.num_programs > cus) p.num_programs = cus;       // (the stream-K workspace is sized for one program per CU)
  p.workspace = workspace;
  const bool skinny_allowed = tile_arg < 0 && knob(knobs().skinny, 1);  // an explicit tile means a tile kernel
  if (skinny_allowed) {
    // at most 64 rows on one side: stream the other operand once (X = small side, Y = streamed side).  65 .. 128 rows
    // against a streamed side of at least 2048: two such launches, 64 rows and the rest - the tile kernels have too
    // few tiles there (flushed do_bench, bf16, tile kernel / two launches: 2048 x 128 x 4096 50.6 / 39.1 us, 8192 x 128 x
    // 8192 117 / 95, 128 x 8192 x 8192 124 / 102; with 256 rows the tiles win, 115 / 147).
    SkinnyArgs sk{};
    sk.K = K; sk.C = (char*)C; sk.a_scale = a_scale; sk.b_scale = b_scale;
    sk.activation = activation; sk.out_dtype = out_dtype; sk.cus = device_info().cus;
    bool use = false, y_kmajor = false, x_kmajor = true;
    int small = 0;
    if (M <= 64 || (M <= 128 && N >= 2048)) {
      sk.X = (const char*)A; sk.Y = (const char*)B; small = M; sk.L = N;
      sk.x_pitch = p.lda; sk.y_pitch = p.ldb; sk.cs = scm; sk.cl = scn;
      sk.aux = aux; sk.aux_ss = aux_sm; sk.aux_sl = aux_sn; sk.aux_dtype = aux_dtype;
      y_kmajor = b_kmajor; use = true;
    } else if (N <= 64 || (N <= 128 && M >= 2048)) {
      sk.X = (const char*)B; sk.Y = (const char*)A; small = N; sk.L = M;
      sk.x_pitch = p.ldb; sk.y_pitch = p.lda; sk.cs = scn; sk.cl = scm;
      sk.aux = aux; sk.aux_ss = aux_sn; sk.aux_sl = aux_sm; sk.aux_dtype = aux_dtype;
      y_kmajor = true; x_kmajor = b_kmajor; use = true;
    }
    if (use) {
      SkinnyArgs part[2] = {sk, sk};
      part[0].S = small < 64 ? small : 64;
      part[1].S = small - part[0].S;
      // (the second part starts 64 rows of X further: K-contiguous rows 64 pitches, S-contiguous rows 64 elements on)
      part[1].X = sk.X + (x_kmajor ? 64 * sk.x_pitch : (int64_t)64 * es);
      part[1].C = sk.C + 64 * sk.cs * elem_size(out_dtype);
      if (aux) part[1].aux = (const char*)aux + 64 * sk.aux_ss * elem_size(aux_dtype);
      const int nparts = part[1].S > 0 ? 2 : 1;
      bool ok = true;
      for (int i = 0; i < nparts; i++) ok = ok && gemm_skinny_ok(part[i], y_kmajor, x_kmajor, es);
      if (ok) {
        for (int i = 0; i < nparts; i++) {
          const int rc = gemm_skinny_launch(part[i], in_dtype, y_kmajor, x_kmajor, stream);
          if (rc != 0) return rc;
        }
        return MI355_OK;
      }
    }
  }
  if (is8 && b_kmajor && !aux && gemm8_skinny_ok(p) && skinny_allowed) return gemm8_skinny_launch(p, in_dtype == MI355_F8E5M2, stream);
  if (is8 && mixed_rows > 0) return gemm_wave128_f8_mixed_launch(p, mixed_rows, in_dtype == MI355_F8E5M2, stream);
  if (is8 && tile == 6 && (p.tile_m == 192 || p.tile_m == 128 || w128_ok)) return gemm_wave128_f8_launch(p, in_dtype == MI355_F8E5M2, b_kmajor, stream);
  if (is8) return gemm8_launch(p, in_dtype == MI355_F8E5M2, b_kmajor, tile, stream);
  // 6: four waves, 128x128 of C per wave from 16x16x32 MFMAs (whole tiles)
  // (a tile height of 192 / 128 rows was set above only after gemm_wave128_192_ok had accepted the shape for it)
  if (mixed_rows > 0 && !is8) return gemm_wave128_mixed_launch(p, mixed_rows, in_dtype == MI355_BF16, b_kmajor, stream);
  if (tile == 6 && (p.tile_m == 192 || p.tile_m == 128 || gemm_wave128_ok(p, b_kmajor, in_dtype))) return gemm_wave128_launch(p, in_dtype == MI355_BF16, b_kmajor, stream);
  return gemm16_launch(p, in_dtype == MI355_BF16, b_kmajor, tile, stream);
}

int mi355_gemm(const void* A, const void* B, void* C, int M, int N, int K,
               int64_t sam, int64_t sak, int64_t sbk, int64_t sbn, int64_t scm, int64_t scn,
               int in_dtype, int out_dtype, const float* a_scale, const float* b_scale,
               int activation, void* stream_) {
  return gemm_impl(A, B, C, M, N, K, sam, sak, sbk, sbn, scm, scn, in_dtype, out_dtype, a_scale, b_scale,
                   activation, nullptr, 0, 0, 0, -1, 0, stream_);
}

int mi355_gemm_tuned(const void* A, const void* B, void* C, int M, int N, int K,
                     int64_t sam, int64_t sak, int64_t sbk, int64_t sbn, int64_t scm, int64_t scn,
                     int in_dtype, int out_dtype, const float* a_scale, const float* b_scale,
                     int activation, int tile, int group_m, void* stream_) {
  if (tile < -1 || tile > 6 || group_m < 0) return MI355_EINVAL;
  return gemm_impl(A, B, C, M, N, K, sam, sak, sbk, sbn, scm, scn, in_dtype, out_dtype, a_scale, b_scale,
                   activation, nullptr, 0, 0, 0, tile, group_m, stream_);
}

int mi355_gemm_splitk(const void* A, const void* B, void* C, int M, int N, int K,
                      int64_t sam, int64_t sak, int64_t sbk, int64_t sbn, int64_t scm, int64_t scn,
                      int in_dtype, int out_dtype, const float* a_scale, const float* b_scale,
                      int activation, int splits, void* workspace, size_t workspace_bytes, void* stream_) {
  if (!A || !B || !C || M <= 0 || N <= 0 || K <= 0 || splits < 0) return MI355_EINVAL;
  if (activation != MI355_ACT_NONE && activation != MI355_ACT_LEAKY_RELU) return MI355_EINVAL;
  if (in_dtype < MI355_F16 || in_dtype > MI355_F32) return MI355_EDTYPE;
  if (out_dtype < MI355_F16 || out_dtype > MI355_F32) return MI355_EDTYPE;
  if (!device_info().gfx950) return MI355_EDEVICE;
  const int es = elem_size(in_dtype), vec = 16 / es;
  // what the tile kernels ask of the operands (as in mi355_gemm); anything else, or nothing to split: the plain call
  const bool a_ok = sak == 1 && sam % vec == 0 && sam >= K && aligned(A, 16) && K % vec == 0;
  const bool b_kmajor = sbk == 1 && sbn % vec == 0 && sbn >= K && aligned(B, 16);
  const bool is32 = in_dtype == MI355_F32;   // (fp32 operands: the fp32 MFMAs, K-major B only)
  const bool b_nmajor = !is32 && sbn == 1 && sbk % vec == 0 && sbk >= (N + vec - 1) / vec * vec && aligned(B, 16);
  const bool pitch_ok = (int64_t)sam * es < (1 << 23) && (b_kmajor ? (int64_t)sbn * es < (1 << 23) : (int64_t)sbk * es < (1 << 26));
  const int64_t k_bytes = (int64_t)K * es;
  const int ksteps = (int)((k_bytes + 63) / 64);
  const int cus = device_info().cus > 0 ? device_info().cus : 256;
  if (splits == 0) {
    // a workgroup per CU, at least sixteen K steps each, at most 32 slices to add up; nothing to gain from half a round
    // of tiles on or below 64 K steps (measured: see ops.py::_splitk_splits)
    const long tiles = (long)((M + 127) / 128) * ((N + 127) / 128);
    splits = tiles * 2 > cus || ksteps < 64 ? 1 : (int)std::min<long>(std::min<long>(cus / tiles, ksteps / 16), 32);
    // (fp32: bound by the fp32 MFMA rate alone, 2048 cycles per K step of a 128x128 tile - whatever puts more CUs to work
    // wins, down to eight K steps a slice; 1024^3: 74 -> 24 us)
    if (is32) splits = tiles >= cus || ksteps < 16 ? 1 : (int)std::min<long>(std::min<long>((2 * cus + tiles - 1) / tiles, ksteps / 8), 32);
  }
  const int per = splits >= 2 ? (ksteps + splits - 1) / splits : ksteps;
  const int used = (ksteps + per - 1) / per;   // (no split is left empty)
  if (!(a_ok && (b_kmajor || b_nmajor) && pitch_ok) || used < 2 || knob(knobs().force_strided, 0) != 0)
    return mi355_gemm(A, B, C, M, N, K, sam, sak, sbk, sbn, scm, scn, in_dtype, out_dtype, a_scale, b_scale, activation, stream_);
  if (!workspace || !aligned(workspace, 16) || workspace_bytes < (size_t)used * M * N * sizeof(float)) return MI355_EINVAL;
  hipStream_t stream = (hipStream_t)stream_;
  GemmArgs p{};
  p.A = (const char*)A; p.B = (const char*)B; p.C = (char*)C;
  p.M = M; p.N = N; p.K = K; p.k_bytes = (int)k_bytes;
  p.lda = sam * es;
  p.ldb = (b_kmajor ? sbn : sbk) * es;
  p.group_m = knob(knobs().group_m, 8);
  p.workspace = (float*)workspace;
  const int rc = is32    ? gemm32_splitk_launch(p, used, per * 64, stream)
                 : es == 1 ? gemm8_splitk_launch(p, in_dtype == MI355_F8E5M2, b_kmajor, used, per * 64, stream)
                           : gemm16_splitk_launch(p, in_dtype == MI355_BF16, b_kmajor, used, per * 64, stream);
  if (rc != 0) return rc;
  GemmStridedArgs out{};
  out.C = C; out.M = M; out.N = N; out.scm = scm; out.scn = scn;
  out.a_scale = a_scale; out.b_scale = b_scale; out.activation = activation; out.out_dtype = out_dtype;
  return splitk_reduce_launch(out, (const float*)workspace, used, stream);
}

int mi355_gemm_streamk(const void* A, const void* B, void* C, int M, int N, int K,
                       int64_t sam, int64_t sak, int64_t sbk, int64_t sbn, int64_t scm, int64_t scn,
                       int in_dtype, int out_dtype, const float* a_scale, const float* b_scale,
                       int activation, void* workspace, size_t workspace_bytes, void* stream_) {
  if (!workspace || !aligned(workspace, 16)) return MI355_EINVAL;
  if (workspace_bytes < (size_t)mi355_query(MI355_Q_STREAMK_WORKSPACE_BYTES)) return MI355_EINVAL;
  // partial 256x256 tiles, or fewer than 64 rows on a side (the streaming kernels): the plain call
  const bool whole_tiles = M > 0 && N > 0 && M % 256 == 0 && N % 256 == 0;
  return gemm_impl(A, B, C, M, N, K, sam, sak, sbk, sbn, scm, scn, in_dtype, out_dtype, a_scale, b_scale,
                   activation, nullptr, 0, 0, 0, whole_tiles ? 7 : -1, 0, stream_, (float*)workspace);
}

// ---- stream-K without an allocation anywhere: the partial-tile workspace is a static device array.
// Host code must never use the array's NAME as an address (there it is a host-side stand-in; a kernel
// handed it would fault): the address on each device comes from hipGetSymbolAddress, once per device,
// and only that pointer is passed on.
constexpr int kStaticStreamKPrograms = 256;                                   // one program per CU of an MI355X
constexpr size_t kStaticStreamKBytes = (size_t)kStaticStreamKPrograms * 2 * 256 * 256 * 4;   // 128 MiB
static __device__ __align__(256) unsigned char scratch[kStaticStreamKBytes];

namespace {
constexpr int kMaxDevices = 64;
void* g_scratch_ptr[kMaxDevices];          // per device: each GPU holds its own copy of the array
std::mutex g_scratch_mutex;

int static_scratch(void** out) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= kMaxDevices) return MI355_EDEVICE;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));   // with device `dev` current: that device's copy
    if (e != hipSuccess) return (int)e;
    if (!ptr) return MI355_EDEVICE;
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return MI355_OK;
}
}  // namespace

int mi355_gemm_streamk_static(const void* A, const void* B, void* C, int M, int N, int K,
                              int64_t sam, int64_t sak, int64_t sbk, int64_t sbn, int64_t scm, int64_t scn,
                              int in_dtype, int out_dtype, const float* a_scale, const float* b_scale,
                              int activation, void* stream_) {
  if (!A || !B || !C || M <= 0 || N <= 0 || K <= 0) return MI355_EINVAL;
  // the static array holds two partial tiles for each of at most 256 programs (one per CU)
  const int cus = device_info().cus > 0 ? device_info().cus : 256;
  const int programs = knob(knobs().programs, cus) < cus ? knob(knobs().programs, cus) : cus;
  if (programs > kStaticStreamKPrograms) return MI355_ESCRATCH;
  void* ws = nullptr;
  const int rc = static_scratch(&ws);
  if (rc) return rc;
  const bool whole_tiles = M > 0 && N > 0 && M % 256 == 0 && N % 256 == 0;
  return gemm_impl(A, B, C, M, N, K, sam, sak, sbk, sbn, scm, scn, in_dtype, out_dtype, a_scale, b_scale,
                   activation, nullptr, 0, 0, 0, whole_tiles ? 7 : -1, 0, stream_, (float*)ws);
}

int mi355_gemm_epilogue(const void* A, const void* B, void* C, int M, int N, int K,
                        int64_t sam, int64_t sak, int64_t sbk, int64_t sbn, int64_t scm, int64_t scn,
                        int in_dtype, int out_dtype, const float* a_scale, const float* b_scale,
                        const void* addend, int64_t stride_dm, int64_t stride_dn, int addend_dtype,
                        int activation, int softmax, void* stream_) {
  if (softmax != 0 && softmax != 1) return MI355_EINVAL;
  if (softmax && out_dtype != MI355_F16 && out_dtype != MI355_BF16 && out_dtype != MI355_F32) return MI355_EDTYPE;
  // a row that fits one tile: product, addend, activation and softmax in ONE launch, on the fp32 accumulator,
  // one rounding at the store - what the reference's single tile does
  // (that kernel is one workgroup per 128 rows with operands of any strides, built for the small products of the
  // reference's test, where the single rounding is the point: on time the tiled GEMM plus a softmax launch wins at every
  // size - flushed caches, bf16: 32^3 10.8 against 9.3 us, 128 x 256 x 128 50 / 13, 1024 x 256 x 256 59 / 14, 8192 x 256 x 256
  // 59 / 19, 256 x 256 x 2048 237 / 33 - and takes over beyond 2^18 elements of A by default, MI355_ROWFUSED_MAX_MK)
  const int64_t rowfused_max = (int64_t)knob(knobs().rowfused_max_mk, 1 << 18);
  if (softmax && N <= 256 && (in_dtype == MI355_F16 || in_dtype == MI355_BF16) && (int64_t)M * K <= rowfused_max) {
    if (!A || !B || !C || M <= 0 || N <= 0 || K <= 0) return MI355_EINVAL;
    if (addend && addend_dtype != MI355_F16 && addend_dtype != MI355_BF16 && addend_dtype != MI355_F32) return MI355_EDTYPE;
    if (activation != MI355_ACT_NONE && activation != MI355_ACT_LEAKY_RELU) return MI355_EINVAL;
    if (!device_info().gfx950) return MI355_EDEVICE;
    RowFusedArgs r{A, B, C, nullptr, M, N, K, 0, sam, sak, sbk, sbn, 0, 0, scm, scn, a_scale, b_scale,
                   activation, 1, out_dtype, addend, stride_dm, stride_dn, addend_dtype};
    return gemm_rowfused_launch(r, in_dtype == MI355_BF16, (hipStream_t)stream_);
  }
  int rc = gemm_impl(A, B, C, M, N, K, sam, sak, sbk, sbn, scm, scn, in_dtype, out_dtype, a_scale, b_scale,
                     activation, addend, stride_dm, stride_dn, addend_dtype, -1, 0, stream_);
  if (rc || !softmax) return rc;
  return softmax_rows_launch(C, M, N, scm, scn, out_dtype, (hipStream_t)stream_);
}

int mi355_gemm_chain(const void* A, const void* B, const void* W, void* C, int M, int N, int K, int N2,
                     int64_t sam, int64_t sak, int64_t sbk, int64_t sbn, int64_t swn, int64_t swn2, int64_t scm, int64_t scn,
                     int in_dtype, int out_dtype, const float* a_scale, const float* b_scale,
                     const void* addend, int64_t stride_dm, int64_t stride_dn, int addend_dtype,
                     int activation, int softmax, void* stream_) {
  if (!A || !B || !W || !C || M <= 0 || N <= 0 || K <= 0 || N2 <= 0) return MI355_EINVAL;
  if (softmax != 0 && softmax != 1) return MI355_EINVAL;
  if (activation != MI355_ACT_NONE && activation != MI355_ACT_LEAKY_RELU) return MI355_EINVAL;
  if (in_dtype != MI355_F16 && in_dtype != MI355_BF16) return MI355_EDTYPE;
  if (out_dtype != MI355_F16 && out_dtype != MI355_BF16 && out_dtype != MI355_F32) return MI355_EDTYPE;
  if (addend && addend_dtype != MI355_F16 && addend_dtype != MI355_BF16 && addend_dtype != MI355_F32) return MI355_EDTYPE;
  if (N > 256 || N2 > 256) return MI355_ESHAPE;   // the intermediate row must fit one tile (callers chain two products otherwise)
  if (!device_info().gfx950) return MI355_EDEVICE;
  RowFusedArgs r{A, B, C, W, M, N, K, N2, sam, sak, sbk, sbn, swn, swn2, scm, scn, a_scale, b_scale,
                 activation, softmax, out_dtype, addend, stride_dm, stride_dn, addend_dtype};
  return gemm_rowfused_launch(r, in_dtype == MI355_BF16, (hipStream_t)stream_);
}

int mi355_grouped_gemm(const void* d_a_ptrs, const void* d_b_ptrs, const void* d_c_ptrs,
                       const int32_t* d_sizes, const int32_t* d_lds, int group_size,
                       int dtype, int num_programs, void* stream_) {
  if (!d_a_ptrs || !d_b_ptrs || !d_c_ptrs || !d_sizes || !d_lds || group_size < 0 || num_programs < 0) return MI355_EINVAL;
  if (dtype != MI355_F16 && dtype != MI355_BF16) return MI355_EDTYPE;
  if (!device_info().gfx950) return MI355_EDEVICE;
  if (group_size == 0) return MI355_OK;
  GroupedArgs ga{};
  ga.a_ptrs = (const uint64_t*)d_a_ptrs; ga.b_ptrs = (const uint64_t*)d_b_ptrs; ga.c_ptrs = (const uint64_t*)d_c_ptrs;
  ga.sizes = d_sizes; ga.lds = d_lds; ga.group_size = group_size; ga.out_dtype = dtype;
  const int cus = device_info().cus > 0 ? device_info().cus : 256;
  const int nprog = num_programs > 0 ? num_programs : 2 * cus;
  // groups with at least one 256x256 tile per CU run 256x256 tiles, one program per CU (never more
  // programs than the caller asked for); MI355_GROUPED_BIG_MIN moves the threshold (a huge value = never)
  const int nprog_big = nprog < cus ? nprog : cus;
  ga.big_tiles_min = knob(knobs().grouped_big_min, cus);
  // smallest K of a group of whole 256x256 tiles that the four-wave 16x16-MFMA kernel takes (0 = never)
  ga.wave128_min_k = knob(knobs().grouped_wave128_min_k, 512);
  ga.chunk = knob(knobs().grouped_chunk, 4);
  if (ga.chunk < 1) ga.chunk = 1;
  return gemm16_grouped_launch(ga, dtype == MI355_BF16, nprog, nprog_big, (hipStream_t)stream_);
}

int mi355_mx_gemm(const uint8_t* A, const uint8_t* sA, const uint8_t* B, const uint8_t* sB, void* C,
                  int M, int N, int K, int fmt, int out_dtype,
                  int64_t lda, int64_t ldb, int64_t lds_a, int64_t lds_b, int64_t ldc, void* stream_) {
  if (!A || !sA || !B || !sB || !C || M <= 0 || N <= 0 || K <= 0) return MI355_EINVAL;
  if (fmt != MI355_MXFP4 && fmt != MI355_MXFP8) return MI355_EINVAL;
  if (out_dtype != MI355_F16 && out_dtype != MI355_BF16 && out_dtype != MI355_F32) return MI355_EDTYPE;
  if (!device_info().gfx950) return MI355_EDEVICE;
  if (K % 32 != 0) return MI355_ESHAPE;  // whole scale blocks only
  const int64_t row_bytes = fmt == MI355_MXFP4 ? K / 2 : K;
  if (lda < row_bytes || ldb < row_bytes || lds_a < K / 32 || lds_b < K / 32 || ldc < N) return MI355_ESTRIDE;
  if (lda % 16 || ldb % 16 || !aligned(A, 16) || !aligned(B, 16)) return MI355_ESTRIDE;
  if (lda >= (1 << 23) || ldb >= (1 << 23)) return MI355_ESTRIDE;  // 32-bit offsets inside a 256-row tile
  GemmArgs p{};
  p.A = (const char*)A; p.B = (const char*)B; p.C = (char*)C;
  p.M = M; p.N = N; p.K = K; p.k_bytes = (int)row_bytes;
  p.lda = lda; p.ldb = ldb; p.ldc = ldc; p.scn = 1;
  p.out_dtype = out_dtype;
  p.group_m = knob(knobs().group_m, 8);
  p.c_vec_ok = ldc % 4 == 0 && aligned(C, 16);
  p.lean_ok = knob(knobs().lean_epilogue, 1);
  p.sA = sA; p.sB = sB; p.lds_a = lds_a; p.lds_b = lds_b;
  const int cus = device_info().cus > 0 ? device_info().cus : 256;
  const long tiles256 = (long)((M + 255) / 256) * ((N + 255) / 256);
  int tile = (tiles256 * 2 >= cus) ? (tiles256 % cus == 0 ? 5 : 4) : 1;
  // MXFP4 with whole 256x256 tiles, K at least 1024 and at least half a round of tiles: four waves of
  // scaled 16x16x128 MFMAs (8192^3: 4000-4050 vs 3340-3640 TFLOP/s for the persistent eight-wave kernel)
  // K beyond the last whole group of K steps (four 128-byte steps for MXFP4, eight for MXFP8) is those kernels' tail
  // form, whose steps are not pipelined: one costs about 3.5 (MXFP4) / 7 (MXFP8) steps of the main loop (8192 x 8192 x
  // 8704: MXFP4 3890 vs 3540 TFLOP/s for the eight-wave kernel, MXFP8 2110 vs 2100; x 4608: 3230 vs 3280 and 1740 vs
  // 2040).  It is chosen where the tail is short against the main loop - and wherever the eight-wave kernels cannot take
  // the product at all (K bytes not a multiple of 64: 8192 x 8192 x 8224 ran the one-thread-per-output kernel, 700 ms).
  auto tail_pays = [&](int group_bytes, int cost) {
    const int tail = p.k_bytes % group_bytes;
    if (tail == 0) return true;
    const bool eight_wave_runs = p.k_bytes % 64 == 0 && lds_a % 4 == 0 && lds_b % 4 == 0 && aligned(sA, 4) && aligned(sB, 4);
    return !eight_wave_runs || (int64_t)((tail + 127) / 128) * cost <= (int64_t)(p.k_bytes - tail) / 128;
  };
  // (below half a round of tiles the four-wave kernels still win where K is long - flushed do_bench, four-wave / 128 x 128
  // tiles: MXFP4 2048 x 2048 x 4096 1010 / 745 TFLOP/s, 1024 x 1024 x 4096 240 / 198, MXFP8 2048 x 2048 x 4096 636 / 407,
  // 1536 x 1536 x 2048 278 / 219 - and lose where it is short: MXFP4 2048 x 2048 x 1024 427 / 504, 1024^3 117 / 139)
  const bool enough = tiles256 * 2 >= cus || (tiles256 >= 16 && p.k_bytes >= 1024);
  if (fmt == MI355_MXFP4 && enough && gemm_wave128_mxfp4_ok(p) && tail_pays(512, 9)) tile = 6;
  // (MXFP8 likewise: 2530-2570 vs 2110-2240)
  if (fmt == MI355_MXFP8 && enough && gemm_wave128_mxfp8_ok(p) && tail_pays(1024, 21)) tile = 6;
  // the same kernels on tiles of 128 x 256 wherever those fit one round of CUs (from 16 on): flushed do_bench, best of
  // the other forms / 128-row tiles, MXFP4: 1024^3 141 / 162 TFLOP/s, 2048 x 2048 x 1024 503 / 600, 2048 x 2048 x 4096 1012 /
  // 1309, 1536 x 2048 x 8192 1071 / 1216, 3072 x 2048 x 4096 1661 / 1854, 2304 x 2048 x 8192 1606 / 1795; MXFP8: 92 / 127,
  // 360 / 491, 644 / 856, 627 / 754, 1072 / 1244, 947 / 1120; beyond one round they lose (3072^3, 288 tiles: MXFP4 2084 for
  // the 192-row tiles / 1555, 4096^3 3209 / 2834)
  if ((knobs().tile == UNSET || knobs().tile_m == 128) && gemm_wave128_mx_192_ok(p, fmt == MI355_MXFP4 ? 512 : 1024, 128)) {
    const long tiles128 = (long)(M / 128) * (N / 256);
    const int want = knob(knobs().tile_m, 0);
    if (want == 128 || (want == 0 && tiles128 >= 16 && tiles128 <= cus)) {
      tile = 6;
      p.tile_m = 128;
    }
  }
  // and on tiles of 192 x 256 where those fill the CUs better (as for the 16-bit and fp8 products).  Flushed
  // do_bench, 256-row choice / 192-row tiles, MXFP4: 3072^3 1750 / 2100 TFLOP/s, 4608 x 4096 x 4096 2475 / 2885, 6144^3
  // 3725 / 3970, 1536 x 8192 x 8192 3205 / 3780, 1536 x 2048 x 8192 880 / 1080; MXFP8: 1255 / 1420, 1480 / 1830, 2275 / 2520,
  // 1945 / 2345, 519 / 630; not taken where they fill worse (3840 x 3840 x 4096: 3080 / 2230)
  if ((knobs().tile == UNSET || knobs().tile_m == 192) && p.tile_m == 0 && gemm_wave128_mx_192_ok(p, fmt == MI355_MXFP4 ? 512 : 1024)) {
    auto fill = [&](long t) { return t <= 0 ? 0.0 : (double)t / (double)(((t + cus - 1) / cus) * cus); };
    const long tiles192 = (long)(M / 192) * (N / 256);
    const int want = knob(knobs().tile_m, 0);
    const bool enough192 = tiles192 * 2 >= cus || (tiles192 >= 16 && p.k_bytes >= 1024);
    if (want == 192 || (want == 0 && enough192 && (tile != 6 || fill(tiles192) > fill(tiles256) * 1.1))) {
      tile = 6;
      p.tile_m = 192;
    }
  }
  p.num_programs = knob(knobs().programs, cus);
  // and on both tile heights in one launch, as for the 16-bit and fp8 products
  if (knobs().tile == UNSET && knobs().tile_m == UNSET && N % 256 == 0) {
    const int want = knob(knobs().mixed_rows, -1), group = fmt == MI355_MXFP4 ? 512 : 1024;
    int rows = 0;
    if (want > 0) rows = want;
    else if (want < 0 && tile == 6 && p.tile_m == 0 && tiles256 > cus) rows = mixed_split(M, N / 256, cus);
    if (rows > 0 && gemm_wave128_mx_mixed_ok(p, group, rows)) return gemm_wave128_mx_mixed_launch(p, fmt == MI355_MXFP4 ? 0 : 1, rows, (hipStream_t)stream_);
  }
  tile = knob(knobs().tile, tile);
  return mx_gemm_launch(p, fmt, tile, (hipStream_t)stream_);
}

int mi355_clock_probe(uint64_t* ticks, int duration_us, void* stream_) {
  if (!ticks || !aligned(ticks, 8) || duration_us <= 0 || duration_us > 2000000) return MI355_EINVAL;
  if (!device_info().gfx950 || device_info().wall_clock_khz <= 0) return MI355_EDEVICE;
  const unsigned long long real_ticks = (unsigned long long)duration_us * (unsigned long long)device_info().wall_clock_khz / 1000ull;
  return clock_probe_launch((unsigned long long*)ticks, real_ticks, (hipStream_t)stream_);
}

int mi355_mfma_burn(float* sink, int shape, int random_operands, int iters, int waves_per_simd, void* stream_) {
  if (!sink || !aligned(sink, 4) || shape < MI355_BURN_BF16_32X32X16 || shape > MI355_BURN_MXFP4_16X16X128) return MI355_EINVAL;
  if (iters <= 0 || iters > (1 << 24) || waves_per_simd < 1 || waves_per_simd > 2) return MI355_EINVAL;
  if (!device_info().gfx950) return MI355_EDEVICE;
  return mfma_burn_launch(sink, shape, random_operands != 0, iters, waves_per_simd, device_info().cus > 0 ? device_info().cus : 256,
                          (hipStream_t)stream_);
}

int mi355_dequant(const uint8_t* codes, float* out, int64_t n, int fmt, void* stream_) {
  if (!codes || !out || n < 0) return MI355_EINVAL;
  if (fmt < MI355_DEQ_E4M3 || fmt > MI355_DEQ_E8M0) return MI355_EINVAL;
  if (n == 0) return MI355_OK;
  if (n > (int64_t)0x7FFFFFFF * 256) return MI355_ESHAPE;
  return dequant_launch(codes, out, n, fmt, (hipStream_t)stream_);
}

static int attn_common(AttnArgs& p, int Z, int H, int N_CTX, int D, int dtype) {
  if (Z <= 0 || H <= 0 || N_CTX <= 0) return MI355_EINVAL;
  if (dtype != MI355_F16 && dtype != MI355_BF16) return MI355_EDTYPE;
  // head_dim 256 and the padded forms of head dims 16 / 32: the forward kernels of every type and the backward
  const bool small = D == 16 || D == 32;
  if (D != 64 && D != 128 && D != 256 && !small) return MI355_ESHAPE;
  if (N_CTX % 128 != 0) return MI355_ESHAPE;
  if (!device_info().gfx950) return MI355_EDEVICE;
  // 16 / 32: the 64-column kernels, which pad with zeros on the fly (loads, LDS tiles and stores know d_real)
  p.Z = Z; p.H = H; p.N = N_CTX; p.D = small ? 64 : D; p.d_real = D;
  return MI355_OK;
}

static bool attn_stride_ok(const int64_t* s, const void* ptr, int D) {
  // rows at most 2^24 elements apart: the kernels address 64 rows of a tile with 32-bit byte offsets
  return s[3] == 1 && s[2] >= D && s[2] < (1 << 24) && s[0] % 8 == 0 && s[1] % 8 == 0 && s[2] % 8 == 0 && aligned(ptr, 16);
}

int mi355_attn_fwd(const void* q, const void* k, const void* v, void* o, float* Mlse,
                   int Z, int H, int N_CTX, int D,
                   const int64_t* sq, const int64_t* sk, const int64_t* sv, const int64_t* so,
                   float sm_scale, int causal, int dtype, void* stream_) {
  if (!q || !k || !v || !o || !Mlse) return MI355_EINVAL;
  AttnArgs p{};
  if (dtype == MI355_F8E5M2 || dtype == MI355_F8E4M3) {
    // fp8 forward: q, k, o with D contiguous, v with N_CTX contiguous (transposed in memory)
    int rc8 = attn_common(p, Z, H, N_CTX, D, MI355_F16);
    if (rc8) return rc8;
    if (!copy_strides(sq, p.sq) || !copy_strides(sk, p.sk) || !copy_strides(sv, p.sv) || !copy_strides(so, p.so))
      return MI355_EINVAL;
    auto rows16 = [&](const int64_t* s, const void* ptr) {
      return s[3] == 1 && s[2] >= D && s[2] < (1 << 24) && s[0] % 16 == 0 && s[1] % 16 == 0 && s[2] % 16 == 0 && aligned(ptr, 16);
    };
    if (!rows16(p.sq, q) || !rows16(p.sk, k) || !rows16(p.so, o)) return MI355_ESTRIDE;
    if (!(p.sv[2] == 1 && p.sv[3] >= N_CTX && p.sv[3] < (1 << 24) && p.sv[0] % 16 == 0 && p.sv[1] % 16 == 0 && p.sv[3] % 16 == 0 && aligned(v, 16)))
      return MI355_ESTRIDE;
    p.q = (const char*)q; p.k = (const char*)k; p.v = (const char*)v; p.o = (char*)o; p.lse = Mlse;
    p.sm_scale = sm_scale; p.causal = causal != 0;
    p.variant = knob(knobs().attn_fwd_variant, 1);  // fp8: four waves, two workgroups per CU (eight waves measured 6-12 % slower)
    return attn_fwd8_launch(p, dtype == MI355_F8E5M2, (hipStream_t)stream_);
  }
  int rc = attn_common(p, Z, H, N_CTX, D, dtype);
  if (rc) return rc;
  if (!copy_strides(sq, p.sq) || !copy_strides(sk, p.sk) || !copy_strides(sv, p.sv) || !copy_strides(so, p.so))
    return MI355_EINVAL;
  if (!attn_stride_ok(p.sq, q, D) || !attn_stride_ok(p.sk, k, D) || !attn_stride_ok(p.sv, v, D) ||
      !attn_stride_ok(p.so, o, D))
    return MI355_ESTRIDE;
  p.q = (const char*)q; p.k = (const char*)k; p.v = (const char*)v; p.o = (char*)o; p.lse = Mlse;
  p.sm_scale = sm_scale; p.causal = causal != 0;
  // eight waves (256 query rows) per K/V stream halve the L2 -> LDS traffic.  Under the causal mask
  // their row ranges are uneven, which the persistent form (4) evens out by pairing long and short
  // query blocks per program; without a mask the one-item-per-workgroup form (2) is the faster one.
  p.variant = knob(knobs().attn_fwd_variant, causal ? 4 : 2);
  p.num_programs = knob(knobs().attn_programs, device_info().cus > 0 ? device_info().cus : 256);
  // 5: four waves of 64 query rows, 16x16x32 MFMAs, software pipelined inside the wave (head_dim 128)
  if (p.variant == 5 && attn_fwd_pipe_ok(p)) return attn_fwd_pipe_launch(p, dtype == MI355_BF16, (hipStream_t)stream_);
  return attn_fwd_launch(p, dtype == MI355_BF16, (hipStream_t)stream_);
}

int mi355_attn_bwd_preprocess(const void* o, const void* d_o, float* delta,
                              int Z, int H, int N_CTX, int D, const int64_t* stride, int dtype, void* stream_) {
  if (!o || !d_o || !delta) return MI355_EINVAL;
  AttnArgs p{};
  int rc = attn_common(p, Z, H, N_CTX, D, dtype);
  if (rc) return rc;
  if (!copy_strides(stride, p.so)) return MI355_EINVAL;
  if (!attn_stride_ok(p.so, o, D) || !aligned(d_o, 16)) return MI355_ESTRIDE;
  p.o = (char*)o; p.d_o = (const char*)d_o; p.delta = delta;
  // delta is written through the non-const alias below
  p.lse = delta;
  return attn_bwd_pre_launch(p, dtype == MI355_BF16, (hipStream_t)stream_);
}

int mi355_attn_bwd(const void* q, const void* k, const void* v, const void* d_o,
                   const float* Mlse, const float* delta, void* dq, void* dk, void* dv,
                   int Z, int H, int N_CTX, int D, const int64_t* stride,
                   float sm_scale, int causal, int dtype, void* stream_) {
  if (!q || !k || !v || !d_o || !Mlse || !delta || !dq || !dk || !dv) return MI355_EINVAL;
  AttnArgs p{};
  int rc = attn_common(p, Z, H, N_CTX, D, dtype);
  if (rc) return rc;
  if (!copy_strides(stride, p.sq)) return MI355_EINVAL;
  if (!attn_stride_ok(p.sq, q, D) || !aligned(k, 16) || !aligned(v, 16) || !aligned(d_o, 16) ||
      !aligned(dq, 16) || !aligned(dk, 16) || !aligned(dv, 16) || !aligned(Mlse, 16) || !aligned(delta, 16))
    return MI355_ESTRIDE;
  p.q = (const char*)q; p.k = (const char*)k; p.v = (const char*)v; p.d_o = (const char*)d_o;
  p.lse = const_cast<float*>(Mlse); p.delta = delta;
  p.dq = (char*)dq; p.dk = (char*)dk; p.dv = (char*)dv;
  p.sm_scale = sm_scale; p.causal = causal != 0;
  return attn_bwd_launch(p, dtype == MI355_BF16, (hipStream_t)stream_);
}

}  // extern "C"

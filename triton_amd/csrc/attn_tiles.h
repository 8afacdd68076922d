// LDS tiles of the attention kernels: [rows][D * 2 bytes] of fp16/bf16, filled by direct
// global->LDS loads and read both row-wise (ds_read_b128, MFMA operand with the row on the lane
// axis) and transposed (ds_read_b64_tr_b16, MFMA operand with the column on the lane axis).
//
// One XOR swizzle of the 16-byte chunk index serves both patterns on the 64-bank (256 bytes per
// sweep) LDS:
//   D = 128, 256 (256- / 512-byte rows):  chunk ^= ((row & 3) << 2) | ((row >> 2) & 3)
//   D =  64 (128-byte rows):  chunk ^= (((row >> 1) & 1) << 2) | ((row >> 2) & 3)
// Row-wise reads are served 16 lanes (16 consecutive rows, one logical chunk) at a time: the XOR
// value is a bijection of row & 15 (for 128-byte rows together with the half-sweep bit row & 1),
// so the 16 lanes hit 16 different 16-byte slots.  Transpose reads are served 32 lanes at a time:
// 4 consecutive rows x 64 bytes; the two low row bits (for 128-byte rows: bit 1, bit 0 being the
// half-sweep) select different 64-byte groups, so the 32 lanes cover all banks once.
#pragma once
#include "common.h"

namespace mi355 {

template <int RB>
__device__ __forceinline__ int tile_swz(int row) {
  // rows of 256 bytes or more start on a bank-sweep boundary: the same four XOR bits serve both
  if constexpr (RB >= 256) return ((row & 3) << 2) | ((row >> 2) & 3);
  else return (((row >> 1) & 1) << 2) | ((row >> 2) & 3);
}

// x ^ IMM as an instruction the optimiser neither hoists out of the key/value loop nor keeps
// alive across it: one VALU op per fragment address instead of a register per (k-step, column
// block) combination.
template <int IMM>
__device__ __forceinline__ unsigned xor_imm(unsigned x) {
  if constexpr (IMM == 0) return x;
  unsigned r = x;
#if MI355_DEVICE_PASS
  asm volatile("v_xor_b32 %0, %1, %2" : "=v"(r) : "i"(IMM), "v"(x));
#endif
  return r;
}

// Direct-load geometry of a [ROWS][RB] tile copied by NW waves: one wave instruction moves
// 1024 / RB rows; lane -> (row, physical chunk); the SOURCE chunk is the swizzled one.
template <int RB, int ROWS, int NW>
struct AttnTile {
  static constexpr int CPR = RB / 16, RPI = 1024 / RB;
  static constexpr int BYTES = ROWS * RB;
  static constexpr int INST = BYTES / 1024 / NW;
  static_assert(INST >= 1, "tile too small for this wave count");
  // byte offset of the lane's source chunk from the tile's first row
  __device__ static int64_t off(int64_t pitch, int wave, int lane, int i) {
    int r = (i * NW + wave) * RPI + lane / CPR;
    int lc = (lane % CPR) ^ tile_swz<RB>(r);
    return (int64_t)r * pitch + lc * 16;
  }
  // the lane's source chunk lies inside the first `row_bytes` bytes of its row (rows narrower than RB: the rest of
  // the tile is zero-filled once and never loaded)
  __device__ static bool chunk_present(int wave, int lane, int i, int row_bytes) {
    int r = (i * NW + wave) * RPI + lane / CPR;
    int lc = (lane % CPR) ^ tile_swz<RB>(r);
    return lc * 16 < row_bytes;
  }
  __device__ static const char* src(const char* base, int64_t pitch, int wave, int lane, int i) {
    return base + off(pitch, wave, lane, i);
  }
};

// Zero the `bytes` of LDS at `base` with all `nthreads` threads of the workgroup (padded tiles: the chunks that no
// load ever writes must read as zeros); the caller synchronises afterwards.
__device__ __forceinline__ void lds_zero(LDS_PTR(char) base, int bytes, int tid, int nthreads) {
  for (int o = tid * 16; o < bytes; o += nthreads * 16) *(LDS_PTR(i32x4))(base + o) = i32x4{0, 0, 0, 0};
}

// Row-wise operand read.  Lane (l32 = lane % 32, g = lane / 32) of MFMA k-step ks reads chunk
// 2*ks + g of row l32 (+ 32 per sub-tile, which leaves the swizzle unchanged):
//   address = base + rowb + (xk ^ (32 * ks)),   rowb = l32 * RB,  xk = (g ^ swz(l32)) << 4
template <int RB>
struct RowRead {
  unsigned rowb, xk;
  __device__ RowRead(int l32, int g) : rowb(l32 * RB), xk((g ^ tile_swz<RB>(l32)) << 4) {}
  template <int KS>
  __device__ __forceinline__ unsigned addr(unsigned base) const { return base + rowb + xor_imm<KS * 32>(xk); }
};

// Transposed operand read.  Lane i16 = lane % 16 of 16-lane group q4 = lane / 16 (g = q4 / 2)
// addresses row R0 + 4*g + i16/4 (R0 = 16*t + 8*h, a multiple of 8) and the 8-byte piece that
// holds columns 32*c + 16*(q4 & 1) + 4*(i16 & 3) .. +3:
//   address = base + R0 * RB + (tl ^ ((c << 6) | (h << 5)))
// with everything lane dependent folded into tl (the XOR touches only the chunk bits 4..7).
template <int RB>
struct TrRead {
  unsigned tl;
  __device__ TrRead(int i16, int q4) {
    const int g = q4 >> 1, x = i16 >> 2, e = 2 * (q4 & 1) + ((i16 & 3) >> 1);
    const int xs = RB >= 256 ? x : (x >> 1);
    tl = (4 * g + x) * RB + (xs << 6) + ((e ^ g) << 4) + (i16 & 1) * 8;
  }
  template <int C, int H>
  __device__ __forceinline__ unsigned addr(unsigned base) const { return base + xor_imm<(C << 6) | (H << 5)>(tl); }
};

// A wave's result tile of 32 rows x W columns (each element times `scale`) to global memory through 32 * W
// elements of LDS that belong to this wave alone (`lds_w`), for accumulators that hold the tile TRANSPOSED: the
// 32x32 MFMA tile c has the tile's columns 32 c .. 32 c + 31 as its rows, so lane (l32, g) owns row l32 and, in
// register quad rg, the columns 32 c + 8 rg + 4 g .. + 3.  Stores straight from those registers are 64 pieces of 8
// bytes in 32 different rows per instruction, and at one request per piece the memory pipeline of the CU is busy for
// about 8000 cycles per 256 x 128 tile (a twentieth of the forward's 4096-key item, a tenth of a 1024-key one).
// Written to LDS row-wise (16-byte chunks XOR-ed with the row, so that the 8-byte writes of 32 rows spread over the
// banks) and read back 16 bytes per lane, a store instruction covers whole rows.  No barrier inside: only this wave
// touches the buffer and a wave's LDS accesses execute in order - but the CALLER makes sure that nobody else still
// reads or loads into that part of LDS.  PAD: only the first `cols_valid` columns (a multiple of 8) exist in memory.
template <typename S, int W, bool PAD>
__device__ __forceinline__ void store_rows_transposed(const f32x16 (&acc)[W / 32], float scale, unsigned lds_w, char* grow0,
                                                      int64_t gpitch, int rows_valid, int cols_valid, int lane) {
  constexpr int RB = W * 2, CPR = RB / 16, WT = W / 32;
  constexpr int SWEEP = RB >= 256 ? 1 : 256 / RB;   // rows per 256 bytes (one pass over the 64 banks)
  typedef __attribute__((ext_vector_type(4))) S S4;
  const int l32 = lane & 31, g = lane >> 5;
  const unsigned wbase = lds_w + l32 * RB + g * 8, wswz = (l32 / SWEEP) & (CPR - 1);
#pragma unroll
  for (int c = 0; c < WT; c++)
#pragma unroll
    for (int rg = 0; rg < 4; rg++) {
      S4 v;
#pragma unroll
      for (int e = 0; e < 4; e++) v[e] = (S)(acc[c][rg * 4 + e] * scale);
      *(LDS_PTR(S4))(uintptr_t)(wbase + (((4 * c + rg) ^ wswz) * 16)) = v;
    }
  asm volatile("" ::: "memory");
#pragma unroll
  for (int k = 0; k < CPR / 2; k++) {
    const int f = k * 64 + lane, row = f / CPR, chunk = f % CPR;
    const i32x4 v = *(LDS_PTR(i32x4))(uintptr_t)(lds_w + row * RB + ((chunk ^ ((row / SWEEP) & (CPR - 1))) * 16));
    if (row < rows_valid && (!PAD || chunk * 8 < cols_valid)) *(i32x4*)(grow0 + (int64_t)row * gpitch + chunk * 16) = v;
  }
}

}  // namespace mi355

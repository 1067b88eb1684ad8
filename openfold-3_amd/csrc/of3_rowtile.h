// Row tiles: the building block of the kernels that work on the single representation
// ([rows][384] bf16 tensors): 32 rows in an LDS tile, 32 x 32 output tiles with K = 384 whose
// weight operands come straight from global memory.
#pragma once

#include "of3_device.h"

namespace of3 {
namespace rowtile {

constexpr int kK = 384;          // c_s = H * D: reduction length of both linear stages
constexpr int kChunks = kK / 8;  // 16-byte chunks per position

__device__ __forceinline__ float xhalf(float v) { return __shfl_xor(v, 32, 64); }

// LDS tile [32 positions][kChunks]: chunk index XOR position in its low four bits (the 16 lanes
// of a read phase hold 16 consecutive positions at one chunk index and must hit 16 bank windows;
// a row is 768 bytes = 3 windows of 256, so without the key they would all hit the same one)
__device__ __forceinline__ int act_slot(int pos, int chunk) { return pos * kChunks + ((chunk & ~15) | ((chunk ^ pos) & 15)); }

// rows pos0 .. pos0+31 of src (kK channels per row, rows row_stride elements apart) into the LDS
// tile; with LN, normalised (statistics in fp32, result rounded to bf16 as the reference's
// LayerNorm output).  Wave w handles rows 8w .. 8w+7, four at a time: 16 lanes per row, three
// 16-byte chunks per lane, row sums by DPP lane permutations (no LDS traffic).  Rows past n_rows
// repeat the last one (never stored by the callers).
template <bool LN>
__device__ __forceinline__ void fill_tile(u32x4_t* act, const bf16_t* __restrict__ src, long row_stride, long pos0, long n_rows,
                                          const bf16_t* __restrict__ ln_w, const bf16_t* __restrict__ ln_b, int wave,
                                          int lane) {
  static_assert(kChunks == 48, "three chunks per lane, 16 lanes per row");
  const int g = lane >> 4, li = lane & 15;
  u32x4_t wpk[3], bpk[3];
  if (LN) {
#pragma unroll
    for (int c = 0; c < 3; ++c) {
      wpk[c] = *reinterpret_cast<const u32x4_t*>(ln_w + 8 * (li + 16 * c));
      bpk[c] = *reinterpret_cast<const u32x4_t*>(ln_b + 8 * (li + 16 * c));
    }
  }
  u32x4_t raw[2][3];
#pragma unroll
  for (int it = 0; it < 2; ++it) {
    long row = pos0 + 8 * wave + 4 * it + g;
    row = row < n_rows ? row : n_rows - 1;
#pragma unroll
    for (int c = 0; c < 3; ++c) raw[it][c] = *reinterpret_cast<const u32x4_t*>(src + row * row_stride + 8 * (li + 16 * c));
  }
#pragma unroll
  for (int it = 0; it < 2; ++it) {
    const int pos = 8 * wave + 4 * it + g;
    if (LN) {
      float x[3][8];
      float s = 0.f;
#pragma unroll
      for (int c = 0; c < 3; ++c) {
        unpack8(raw[it][c], x[c]);
#pragma unroll
        for (int i = 0; i < 8; ++i) s += x[c][i];
      }
      const float mean = group_sum<16>(s) * (1.f / kK);
      float q = 0.f;
#pragma unroll
      for (int c = 0; c < 3; ++c)
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          x[c][i] -= mean;
          q += x[c][i] * x[c][i];
        }
      const float rstd = __builtin_amdgcn_rsqf(group_sum<16>(q) * (1.f / kK) + kLnEps);
#pragma unroll
      for (int c = 0; c < 3; ++c) {
        float w[8], bb[8];
        unpack8(wpk[c], w);
        unpack8(bpk[c], bb);
#pragma unroll
        for (int i = 0; i < 8; ++i) x[c][i] = x[c][i] * rstd * w[i] + bb[i];
        raw[it][c] = pack8(x[c]);
      }
    }
#pragma unroll
    for (int c = 0; c < 3; ++c) act[act_slot(pos, li + 16 * c)] = raw[it][c];
  }
}

// 32 x 32 output tile with K = kK, added to `acc`: `w_row` points at the weight row this lane feeds (or is null
// for a zero row), positions come from the LDS tile.  WEIGHTS_ARE_A: result lane (position l32,
// half lh) holds w-rows 16*lh + v (the caller dealt the rows by rowperm16); otherwise lane
// (w-row l32, half lh) holds positions 8*(v/4) + 4*lh + (v%4).
template <bool WEIGHTS_ARE_A>
__device__ __forceinline__ f32x16_t tile_product(const u32x4_t* act, const bf16_t* __restrict__ w_row, int l32, int lh,
                                                 f32x16_t acc = zero16()) {
  // the lane's whole weight row half (24 chunks) is requested before the first MFMA: one trip to
  // L2 per tile instead of one per k-step
  u32x4_t w[kK / 16];
#pragma unroll
  for (int s = 0; s < kK / 16; ++s) {
    w[s] = u32x4_t{0u, 0u, 0u, 0u};
    if (w_row) w[s] = *reinterpret_cast<const u32x4_t*>(w_row + 16 * s + 8 * lh);
  }
#pragma unroll
  for (int s = 0; s < kK / 16; ++s) {
    const u32x4_t x = act[act_slot(l32, 2 * s + lh)];
    acc = WEIGHTS_ARE_A ? mfma_32x32x16(w[s], x, acc) : mfma_32x32x16(x, w[s], acc);
  }
  return acc;
}

// 16 consecutive bf16 values starting at element `first` of a row of `n` valid elements, packed
// as they are; elements at or past n read as zero
__device__ __forceinline__ void load16_raw(const bf16_t* __restrict__ row, int first, int n, bool vec_ok, u32x4_t (&out)[2]) {
  if (vec_ok && first + 16 <= n) {
    out[0] = *reinterpret_cast<const u32x4_t*>(row + first);
    out[1] = *reinterpret_cast<const u32x4_t*>(row + first + 8);
  } else {
#pragma unroll
    for (int w = 0; w < 8; ++w) {
      const uint32_t lo = first + 2 * w < n ? row[first + 2 * w] : 0u;
      const uint32_t hi = first + 2 * w + 1 < n ? row[first + 2 * w + 1] : 0u;
      out[w >> 2][w & 3] = lo | (hi << 16);
    }
  }
}

}  // namespace rowtile
}  // namespace of3

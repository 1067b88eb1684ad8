// Triangle-attention output pass (attention.py:288-302 plus the caller's residual add of
// base_blocks.py:364-378 when requested):
//     out = [x +] (o * sigmoid(LayerNorm(x) Wg^T)) Wo^T
// o is the flash kernel's [b][i][j][H*D] output in the module frame; x / out are addressed
// through the PairView (transposed for the ending node).  The gate is recomputed from x
// rather than stored by the input pass (one z-sized write and read less).
//
// HBM bound: reads o and x once, writes out once.  Two MFMA passes per 128-position tile:
// gate tile -> multiplied into the o tile in LDS in place -> output projection.
#include "of3_device.h"
#include "of3_kernels.h"
#include "of3_launch.h"

namespace of3 {

namespace {

template <int C, int HD>
__global__ __launch_bounds__(512) void triattn_out_kernel(TriattnOutArgs p, int tiles_per_row, int total_tiles) {
  static_assert(C == HD, "o tile shares the x tile geometry");
  constexpr int NCH = C / 8;
  constexpr int LPP = NCH;
  constexpr int PPI = 64 / LPP;
  constexpr int TP = 128;
  constexpr int NW = 8;                  // waves per work-group (two per SIMD)
  constexpr int LN_ITERS = (TP / NW) / PPI;
  constexpr int KS = C / 16;
  constexpr int NOT = C / 32;
  constexpr int WPG = NW / NOT;
  constexpr int TPW = 4 / WPG;

  __shared__ u32x4_t xtile[TP * NCH];  // LayerNorm(x), bf16
  __shared__ u32x4_t otile[TP * NCH];  // o, then o * gate
  __shared__ u32x4_t rtile[TP * NCH];  // x as loaded: the residual of the output phase

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63, l32 = lane & 31, lh = lane >> 5;
  const int ln_chunk = lane % LPP, ln_pp = lane / LPP;

  float lw[8], lb[8];
  load_affine8(p.ln_w, ln_chunk, lw);
  load_affine8(p.ln_b, ln_chunk, lb);

  const int ot = wave % NOT;
  const int t0 = (wave / NOT) * TPW;
  u32x4_t wg[KS], wo[KS];
  {
    const int row = 32 * ot + rowperm16(l32);
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      wg[s] = *reinterpret_cast<const u32x4_t*>(p.w_g + row * C + 16 * s + 8 * lh);
      wo[s] = *reinterpret_cast<const u32x4_t*>(p.w_o + row * HD + 16 * s + 8 * lh);
    }
  }

  const int N = p.N;
  const int tiles_per_batch = N * tiles_per_row;

  // The loads of a tile are issued one tile ahead (right after the previous tile's values have
  // been consumed by the LayerNorm phase) and travel under that tile's two MFMA phases.
  u32x4_t xraw[LN_ITERS], oraw[LN_ITERS];
  auto load_tile = [&](int tile_id) {
    const int b = tile_id / tiles_per_batch;
    const int rem = tile_id - b * tiles_per_batch;
    const int i = rem / tiles_per_row;
    const int j0 = (rem - i * tiles_per_row) * TP;
    const bf16_t* xrow = p.x + b * p.x_view.stride_b + i * p.x_view.stride_r;
    const bf16_t* orow = p.o + ((size_t)b * N + i) * N * HD;
#pragma unroll
    for (int it = 0; it < LN_ITERS; ++it) {
      const int j = j0 + wave * (TP / NW) + it * PPI + ln_pp;
      u32x4_t vx = {0u, 0u, 0u, 0u}, vo = {0u, 0u, 0u, 0u};
      if (j < N) {
        vx = *reinterpret_cast<const u32x4_t*>(xrow + j * p.x_view.stride_k + 8 * ln_chunk);
        vo = *reinterpret_cast<const u32x4_t*>(orow + (size_t)j * HD + 8 * ln_chunk);
      }
      xraw[it] = vx;
      oraw[it] = vo;
    }
  };
  if ((int)blockIdx.x < total_tiles) load_tile(blockIdx.x);

  for (int tile_id = blockIdx.x; tile_id < total_tiles; tile_id += gridDim.x) {
    const int b = tile_id / tiles_per_batch;
    const int rem = tile_id - b * tiles_per_batch;
    const int i = rem / tiles_per_row;
    const int j0 = (rem - i * tiles_per_row) * TP;
    bf16_t* outrow = p.out + b * p.x_view.stride_b + i * p.x_view.stride_r;

    // ---- LayerNorm of this tile's values, then the next tile's loads
#pragma unroll
    for (int it = 0; it < LN_ITERS; ++it) {
      const int pos = wave * (TP / NW) + it * PPI + ln_pp;
      const int slot = tile_slot<NCH, 0>(pos, ln_chunk);
      xtile[slot] = layer_norm_chunk<C>(xraw[it], lw, lb);
      rtile[slot] = xraw[it];
      otile[slot] = oraw[it];
    }
    __syncthreads();
    if (tile_id + (int)gridDim.x < total_tiles) load_tile(tile_id + gridDim.x);

    // ---- gate: lane owns gate channels 32*ot + 16*lh + v of position 32*t + l32
#pragma unroll
    for (int tt = 0; tt < TPW; ++tt) {
      const int pos = 32 * (t0 + tt) + l32;
      f32x16_t acc = zero16();
#pragma unroll
      for (int s = 0; s < KS; ++s) acc = mfma_32x32x16(wg[s], xtile[tile_slot<NCH, 0>(pos, 2 * s + lh)], acc);
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        const int slot = tile_slot<NCH, 0>(pos, 4 * ot + 2 * lh + half);
        float ov[8];
        unpack8(otile[slot], ov);
#pragma unroll
        for (int v = 0; v < 8; ++v) ov[v] *= sigmoidf_fast(acc[8 * half + v]);
        otile[slot] = pack8(ov);
      }
    }
    __syncthreads();

    // ---- output projection (+ residual)
#pragma unroll
    for (int tt = 0; tt < TPW; ++tt) {
      const int pos = 32 * (t0 + tt) + l32;
      f32x16_t acc = zero16();
#pragma unroll
      for (int s = 0; s < KS; ++s) acc = mfma_32x32x16(wo[s], otile[tile_slot<NCH, 0>(pos, 2 * s + lh)], acc);
      const int j = j0 + pos;
      if (j < N) {
        const int64_t off = j * p.x_view.stride_k + 32 * ot + 16 * lh;
        float res[16];
#pragma unroll
        for (int v = 0; v < 16; ++v) res[v] = acc[v];
        if (p.add_residual) {
          const u32x4_t r0 = rtile[tile_slot<NCH, 0>(pos, 4 * ot + 2 * lh)];
          const u32x4_t r1 = rtile[tile_slot<NCH, 0>(pos, 4 * ot + 2 * lh + 1)];
          float xr[8];
          unpack8(r0, xr);
#pragma unroll
          for (int v = 0; v < 8; ++v) res[v] += xr[v];
          unpack8(r1, xr);
#pragma unroll
          for (int v = 0; v < 8; ++v) res[8 + v] += xr[v];
        }
        u32x4_t o0, o1;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          o0[q] = pack_bf16(res[2 * q], res[2 * q + 1]);
          o1[q] = pack_bf16(res[8 + 2 * q], res[8 + 2 * q + 1]);
        }
        *reinterpret_cast<u32x4_t*>(outrow + off) = o0;
        *reinterpret_cast<u32x4_t*>(outrow + off + 8) = o1;
      }
    }
    __syncthreads();
  }
}

template <int C, int HD>
hipError_t launch(const TriattnOutArgs& a, hipStream_t stream) {
  auto kern = triattn_out_kernel<C, HD>;
  static int cache[kMaxDevices];
  int grid_cap = 0;
  hipError_t e = per_device(cache, [&](int dev, int* v) { return resident_blocks(kern, 512, dev, v); }, &grid_cap);
  if (e != hipSuccess) return e;
  const int tiles_per_row = (a.N + 127) / 128;
  const long total = (long)a.B * a.N * tiles_per_row;
  const int grid = (int)(total < grid_cap ? total : grid_cap);
  hipLaunchKernelGGL(kern, dim3(grid), dim3(512), 0, stream, a, tiles_per_row, (int)total);
  return hipGetLastError();
}

}  // namespace

hipError_t triattn_out_launch(const TriattnOutArgs& args, int C, int HD, hipStream_t stream) {
  if (C == 128 && HD == 128) return launch<128, 128>(args, stream);
  if (C == 64 && HD == 64) return launch<64, 64>(args, stream);
  return hipErrorInvalidValue;
}

}  // namespace of3

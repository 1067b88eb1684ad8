// Triangle-attention output pass (attention.py:288-302 plus the caller's residual add of
// base_blocks.py:364-378 when requested):
//     out = [x +] (o * sigmoid(LayerNorm(x) Wg^T)) Wo^T
// o is the flash kernel's [b][i][j][H*D] output in the module frame; x / out are addressed
// through the PairView (transposed for the ending node).  The gate is recomputed from x
// rather than stored by the input pass (one z-sized write and read less).
//
// HBM bound: reads o and x once, writes out once.  Two MFMA passes per 128-position tile:
// gate tile -> multiplied into the o tile in LDS in place -> output projection.
// A tile is 128 consecutive positions of the flattened [B][N][N] index space of the module frame, so it
// may run over the end of a row (or of a batch element): a token count off the multiples of 128 costs
// no partly filled tile per row, only one at the very end.
#include "of3_device.h"
#include "of3_kernels.h"
#include "of3_launch.h"

namespace of3 {

namespace {

template <int C, int HD, int MODE>
__global__ __launch_bounds__(512) void triattn_out_kernel(TriattnOutArgs p, uint32_t total_pos, int total_tiles) {
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

  // LayerNorm(x) feeds the gate only: its weight and bias carry the factor -log2(e) of the gate's
  // base-2 exponential, one multiplication per gate value less
  float lw[8], lb[8];
  load_affine8(p.ln_w, ln_chunk, lw);
  load_affine8(p.ln_b, ln_chunk, lb);
#pragma unroll
  for (int e = 0; e < 8; ++e) lw[e] *= -kLog2e, lb[e] *= -kLog2e;

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
  // A tile starts at position p0 = (b0, i0, j0) (wave-uniform: scalar divisions); with N >= 128 it holds
  // positions of at most two rows, whose offsets in the view are scalars, and position d of the tile costs a
  // compare and two selects (of3_tiles.h).
  typedef FlatTile Origin;
  auto tile_origin = [&](int tile_id) { return flat_tile(tile_id, N, p.x_view.stride_b, p.x_view.stride_r); };
  auto view_offset = [&](const Origin& t, int d) -> int64_t {
    return flat_offset<MODE>(t, d, N, p.x_view.stride_b, p.x_view.stride_r, p.x_view.stride_k);
  };

  // The loads of a tile are issued one tile ahead (right after the previous tile's values have
  // been consumed by the LayerNorm phase) and travel under that tile's two MFMA phases.
  u32x4_t xraw[LN_ITERS], oraw[LN_ITERS];
  auto load_tile = [&](int tile_id) {
    const Origin t = tile_origin(tile_id);
    const uint32_t p0 = (uint32_t)tile_id * TP;
#pragma unroll
    for (int it = 0; it < LN_ITERS; ++it) {
      const int d = wave * (TP / NW) + it * PPI + ln_pp;
      u32x4_t vx = {0u, 0u, 0u, 0u}, vo = {0u, 0u, 0u, 0u};
      if (p0 + d < total_pos) {
        vx = *reinterpret_cast<const u32x4_t*>(p.x + view_offset(t, d) + 8 * ln_chunk);
        vo = *reinterpret_cast<const u32x4_t*>(p.o + (size_t)(p0 + d) * HD + 8 * ln_chunk);  // o is [B][N][N][HD]
      }
      xraw[it] = vx;
      oraw[it] = vo;
    }
  };
  if ((int)blockIdx.x < total_tiles) load_tile(blockIdx.x);

  for (int tile_id = blockIdx.x; tile_id < total_tiles; tile_id += gridDim.x) {
    const Origin t = tile_origin(tile_id);
    const uint32_t p0 = (uint32_t)tile_id * TP;

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
        for (int v = 0; v < 8; ++v) ov[v] *= sigmoid_from_scaled(acc[8 * half + v]);
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
      if (p0 + pos < total_pos) {
        bf16_t* outrow = p.out;
        const int64_t off = view_offset(t, pos) + 32 * ot + 16 * lh;
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

template <int C, int HD, int MODE>
hipError_t launch(const TriattnOutArgs& a, hipStream_t stream) {
  auto kern = triattn_out_kernel<C, HD, MODE>;
  static int cache[kMaxDevices];
  int grid_cap = 0;
  hipError_t e = per_device(cache, [&](int dev, int* v) { return resident_blocks(kern, 512, dev, v); }, &grid_cap);
  if (e != hipSuccess) return e;
  const long positions = (long)a.B * a.N * a.N;
  if (positions <= 0 || positions > 0x7fffffffL) return hipErrorInvalidValue;
  const long total = (positions + 127) / 128;
  const int grid = (int)(total < grid_cap ? total : grid_cap);
  hipLaunchKernelGGL(kern, dim3(grid), dim3(512), 0, stream, a, (uint32_t)positions, (int)total);
  return hipGetLastError();
}

}  // namespace

hipError_t triattn_out_launch(const TriattnOutArgs& args, int C, int HD, hipStream_t stream) {
  // a 128-position tile lies in one row (N a multiple of 128), in at most two (N >= 128), or anywhere
  const int mode = args.N % 128 == 0 ? 0 : (args.N >= 128 ? 1 : 2);
  if (C == 128 && HD == 128)
    return mode == 0 ? launch<128, 128, 0>(args, stream) : (mode == 1 ? launch<128, 128, 1>(args, stream) : launch<128, 128, 2>(args, stream));
  if (C == 64 && HD == 64)
    return mode == 0 ? launch<64, 64, 0>(args, stream) : (mode == 1 ? launch<64, 64, 1>(args, stream) : launch<64, 64, 2>(args, stream));
  return hipErrorInvalidValue;
}

}  // namespace of3

// Triangle-multiplication output pass
//     out = [z +] (LayerNorm_out(x) Wz^T) * sigmoid(LayerNorm_in(z) Wg^T)
// (triangular_multiplicative_update.py:498-501; the optional residual is the caller's
// "z = z + update" of base_blocks.py:329-335 fused in).  x arrives channel-major
// [b][c][i][j] from the contraction and is transposed to position-major on its way into
// LDS; the gate is recomputed from z instead of being stored by the input pass, which
// saves one full write and one full read of a z-sized tensor.
//
// HBM bound: reads x and z once, writes out once.
//
// Tiles are 128 positions: the whole 128-wide pieces of every row first, then, when N is not a multiple
// of 128, the remaining columns in pieces of 2^s columns x 128 / 2^s consecutive rows (2^s the smallest
// power of two >= 8 that covers them), so that the ragged end of the rows costs a few tiles per batch
// element rather than one more tile per row.
#include "of3_device.h"
#include "of3_kernels.h"
#include "of3_launch.h"

namespace of3 {

namespace {

template <int C, int CH, bool RAGGED>
__global__ __launch_bounds__(512) void trimul_out_kernel(TrimulOutArgs p, int full_per_row, int tail_shift, int tiles_per_batch,
                                                           int total_tiles) {
  static_assert(C == CH, "position-major x tile shares the z tile geometry");
  constexpr int NCH = C / 8;
  constexpr int LPP = NCH;
  constexpr int PPI = 64 / LPP;
  constexpr int TP = 128;
  constexpr int NW = 8;                  // waves per work-group (two per SIMD)
  constexpr int LN_ITERS = (TP / NW) / PPI;
  constexpr int KS = C / 16;
  constexpr int NOT = C / 32;            // output-channel tiles
  constexpr int WPG = NW / NOT;          // waves sharing one output tile (2 or 4)
  constexpr int TPW = 4 / WPG;           // position tiles per wave
  constexpr int XROUNDS = (CH / 2) * 16 / 512;  // (channel pair, 8-position group) items per thread

  __shared__ u32x4_t ztile[TP * NCH];
  __shared__ u32x4_t xtile[TP * NCH];
  __shared__ u32x4_t rtile[TP * NCH];  // z as loaded: the residual of the output phase

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63, l32 = lane & 31, lh = lane >> 5;
  const int ln_chunk = lane % LPP, ln_pp = lane / LPP;

  float iw[8], ib[8], ow[8], ob[8];
  load_affine8(p.ln_in_w, ln_chunk, iw);
  load_affine8(p.ln_in_b, ln_chunk, ib);
  load_affine8(p.ln_out_w, ln_chunk, ow);
  load_affine8(p.ln_out_b, ln_chunk, ob);
  // LayerNorm_in(z) feeds the gate only: its weight and bias carry the factor -log2(e) of the gate's
  // base-2 exponential, one multiplication per gate value less
#pragma unroll
  for (int e = 0; e < 8; ++e) iw[e] *= -kLog2e, ib[e] *= -kLog2e;

  // A operands: logical output channel of A-row r is 32*ot + rowperm16(r), so that a lane
  // ends up with the 16 consecutive channels 32*ot + 16*lh + v
  const int ot = wave % NOT;
  const int t0 = (wave / NOT) * TPW;
  u32x4_t wz[KS], wgt[KS];
  {
    const int row = 32 * ot + rowperm16(l32);
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      wz[s] = *reinterpret_cast<const u32x4_t*>(p.w_z + row * CH + 16 * s + 8 * lh);
      wgt[s] = *reinterpret_cast<const u32x4_t*>(p.w_g + row * C + 16 * s + 8 * lh);
    }
  }

  const int N = p.N, Np = p.Np;
  // tile -> batch element, first row, first column, log2 of its width (all wave-uniform); the last ragged
  // piece may run past the last row: those positions are left out below
  auto tile_origin = [&](int tile_id, int& b, int& i0, int& j0, int& shift) {
    const TilePlace t = tile_place<RAGGED>(tile_id, N, full_per_row, tail_shift, tiles_per_batch, false);
    b = t.b, i0 = t.i0, j0 = t.j0, shift = t.shift;
  };
  uint32_t* xt32 = reinterpret_cast<uint32_t*>(xtile);

  // The loads of a tile (z row-wise for the gate, x channel-major) are issued one tile ahead,
  // right after the previous tile's values have gone into LDS, and travel under its MFMA phase.
  u32x4_t zraw[LN_ITERS];
  u32x4_t xa[XROUNDS], xb[XROUNDS];
  auto load_tile = [&](int tile_id) {
    int b, i0, j0, shift_rt;
    tile_origin(tile_id, b, i0, j0, shift_rt);
    const int shift = RAGGED ? shift_rt : 7;  // a constant without ragged pieces: di below folds to 0
    const int jmask = (1 << shift) - 1;
    const bf16_t* zrow = p.z + b * p.z_view.stride_b + i0 * p.z_view.stride_r;  // the tile's first row (scalar)
#pragma unroll
    for (int it = 0; it < LN_ITERS; ++it) {
      const int pos = wave * (TP / NW) + it * PPI + ln_pp;
      const int di = RAGGED ? pos >> shift : 0, j = j0 + (RAGGED ? pos & jmask : pos);  // di = 0 in the whole-row pieces
      u32x4_t v = {0u, 0u, 0u, 0u};
      if ((!RAGGED || i0 + di < N) && j < N) v = *reinterpret_cast<const u32x4_t*>(zrow + di * p.z_view.stride_r + j * p.z_view.stride_k + 8 * ln_chunk);
      zraw[it] = v;
    }
#pragma unroll
    for (int rr = 0; rr < XROUNDS; ++rr) {
      const int item = rr * 512 + tid;
      const int cp = item >> 4, pg = item & 15;  // channels 2cp, 2cp+1; positions 8pg..8pg+7: one row, as the width is >= 8
      int i = i0 + (RAGGED ? (8 * pg) >> shift : 0);
      const int j = j0 + (RAGGED ? (8 * pg) & jmask : 8 * pg);  // < Np: the planes are padded to whole 128-wide pieces
      if (RAGGED) i = i < Np ? i : Np - 1;    // rows of a last piece past the end of the plane: any row, never used
      const bf16_t* src = p.x + (((size_t)b * CH + 2 * cp) * Np + i) * Np + j;
      xa[rr] = *reinterpret_cast<const u32x4_t*>(src);
      xb[rr] = *reinterpret_cast<const u32x4_t*>(src + (size_t)Np * Np);
    }
  };
  if ((int)blockIdx.x < total_tiles) load_tile(blockIdx.x);

  for (int tile_id = blockIdx.x; tile_id < total_tiles; tile_id += gridDim.x) {
    int b, i0, j0, shift_rt;
    tile_origin(tile_id, b, i0, j0, shift_rt);
    const int shift = RAGGED ? shift_rt : 7;
    const int jmask = (1 << shift) - 1;
    bf16_t* orow0 = p.out + b * p.z_view.stride_b + i0 * p.z_view.stride_r;  // the tile's first row (scalar)

    // x: transpose into xtile[pos][c] with 4-byte (channel pair) writes
#pragma unroll
    for (int rr = 0; rr < XROUNDS; ++rr) {
      const int item = rr * 512 + tid;
      const int cp = item >> 4, pg = item & 15;
      const int chunk = (2 * cp) >> 3, within = (2 * cp) & 7;  // `within` is even
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const uint32_t ua = xa[rr][e >> 1], ub = xb[rr][e >> 1];
        const uint32_t w = (e & 1) ? ((ua >> 16) | (ub & 0xffff0000u)) : ((ua & 0xffffu) | (ub << 16));
        const int pos = 8 * pg + e;
        xt32[tile_slot<NCH, 0>(pos, chunk) * 4 + (within >> 1)] = w;
      }
    }
    // z: LayerNorm_in -> ztile
#pragma unroll
    for (int it = 0; it < LN_ITERS; ++it) {
      const int pos = wave * (TP / NW) + it * PPI + ln_pp;
      ztile[tile_slot<NCH, 0>(pos, ln_chunk)] = layer_norm_chunk<C>(zraw[it], iw, ib);
      rtile[tile_slot<NCH, 0>(pos, ln_chunk)] = zraw[it];
    }
    __syncthreads();
    if (tile_id + (int)gridDim.x < total_tiles) load_tile(tile_id + gridDim.x);

    // x: LayerNorm_out in place (lane owns one 16-byte chunk of one position)
#pragma unroll
    for (int it = 0; it < LN_ITERS; ++it) {
      const int pos = wave * (TP / NW) + it * PPI + ln_pp;
      const int slot = tile_slot<NCH, 0>(pos, ln_chunk);
      xtile[slot] = layer_norm_chunk<CH>(xtile[slot], ow, ob);
    }
    __syncthreads();

    // ---- matrix phase
#pragma unroll
    for (int tt = 0; tt < TPW; ++tt) {
      const int t = t0 + tt;
      const int pos = 32 * t + l32;
      f32x16_t accu = zero16(), accg = zero16();
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        const u32x4_t bx = xtile[tile_slot<NCH, 0>(pos, 2 * s + lh)];
        const u32x4_t bz = ztile[tile_slot<NCH, 0>(pos, 2 * s + lh)];
        accu = mfma_32x32x16(wz[s], bx, accu);
        accg = mfma_32x32x16(wgt[s], bz, accg);
      }
      const int di = RAGGED ? pos >> shift : 0, j = j0 + (RAGGED ? pos & jmask : pos);
      if ((!RAGGED || i0 + di < N) && j < N) {
        bf16_t* orow = orow0;
        const int64_t off = di * p.z_view.stride_r + j * p.z_view.stride_k + 32 * ot + 16 * lh;
        float res[16];
#pragma unroll
        for (int v = 0; v < 16; ++v) res[v] = accu[v] * sigmoid_from_scaled(accg[v]);
        if (p.add_residual) {
          const u32x4_t r0 = rtile[tile_slot<NCH, 0>(pos, 4 * ot + 2 * lh)];
          const u32x4_t r1 = rtile[tile_slot<NCH, 0>(pos, 4 * ot + 2 * lh + 1)];
          float zr[8];
          unpack8(r0, zr);
#pragma unroll
          for (int v = 0; v < 8; ++v) res[v] += zr[v];
          unpack8(r1, zr);
#pragma unroll
          for (int v = 0; v < 8; ++v) res[8 + v] += zr[v];
        }
        u32x4_t o0, o1;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          o0[q] = pack_bf16(res[2 * q], res[2 * q + 1]);
          o1[q] = pack_bf16(res[8 + 2 * q], res[8 + 2 * q + 1]);
        }
        *reinterpret_cast<u32x4_t*>(orow + off) = o0;
        *reinterpret_cast<u32x4_t*>(orow + off + 8) = o1;
      }
    }
    __syncthreads();  // both tiles are rewritten by the next iteration
  }
}

template <int C, int CH, bool RAGGED>
hipError_t launch(const TrimulOutArgs& a, hipStream_t stream) {
  auto kern = trimul_out_kernel<C, CH, RAGGED>;
  static int cache[kMaxDevices];
  int grid_cap = 0;
  hipError_t e = per_device(cache, [&](int dev, int* v) { return resident_blocks(kern, 512, dev, v); }, &grid_cap);
  if (e != hipSuccess) return e;
  const RaggedTiles t = ragged_tiles(a.N);
  const long total = (long)a.B * t.per_batch;
  if (total > 0x7fffffffL) return hipErrorInvalidValue;
  const int grid = (int)(total < grid_cap ? total : grid_cap);
  hipLaunchKernelGGL(kern, dim3(grid), dim3(512), 0, stream, a, t.full_per_row, t.tail_shift, t.per_batch, (int)total);
  return hipGetLastError();
}

}  // namespace

hipError_t trimul_out_launch(const TrimulOutArgs& args, int C, int CH, hipStream_t stream) {
  const bool ragged = args.N % 128 != 0;
  if (C == 128 && CH == 128) return ragged ? launch<128, 128, true>(args, stream) : launch<128, 128, false>(args, stream);
  if (C == 64 && CH == 64) return ragged ? launch<64, 64, true>(args, stream) : launch<64, 64, false>(args, stream);
  return hipErrorInvalidValue;
}

}  // namespace of3

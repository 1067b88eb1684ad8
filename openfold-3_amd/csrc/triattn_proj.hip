// Triangle-attention input pass: xn = LayerNorm(x), then
//     q = (xn Wq^T) * log2(e)/sqrt(D),  k = xn Wk^T,  v = xn Wv^T     (attention.py:265-286)
//     triangle bias tb[h][q][k] = log2(e) * (xn[q][k] . Wb[h])          (tri_att.py:137-140)
//     mask bias     mb[i][k]    = log2(e) * inf * (mask[i][k] - 1)      (tri_att.py:134)
// written in the layouts the flash kernel consumes: q, k as [b][i][h][j][d]; v transposed
// in panels of 32 keys as [b][i][h][j/32][d][j%32] (one key tile of one head = 2 KB
// contiguous); tb as [b][h][i][j] and mb as [b][i][j] in fp32.  log2(e) is folded
// in so the softmax can use the hardware base-2 exponential.  The PairView makes (i, j)
// walk either the tensor itself (starting node) or its transpose (ending node).
//
// HBM bound (reads x once, writes q, k, v once).  Same structure as the
// triangle-multiplication input pass: 8 waves per work-group, weights resident in registers
// as MFMA A operands, 128-position tiles normalised in registers and staged once in a
// double-buffered LDS tile (one barrier per tile).
//
// Tiles: the whole 128-wide pieces of every row; when N is not a multiple of 128 (RAGGED), the remaining
// columns come in pieces of 32, 64 or 128 columns x 4, 2 or 1 consecutive rows, so that the ragged end
// of the rows costs a tile per four (two) rows instead of one per row.  The last such piece of a batch
// element is moved up to end at the last row (rows computed twice are written twice with the same values).
// Columns are written up to the end of the 32-wide panel that holds the last token, which is as far as
// the attention core reads.
#include "of3_device.h"
#include "of3_kernels.h"
#include "of3_launch.h"

// Waves per work-group of the C = 128 kernel: 8 (two per SIMD, 248 registers) or 16 (four per SIMD,
// 118 registers, one matrix per wave).  Measured at N = 768 inside the block: 126 us against 128 us,
// stand-alone 150 against 158: more waves in flight do not help this pass, the shipped form is 8.
#ifndef OF3_TP_WAVES
#define OF3_TP_WAVES 8
#endif

namespace of3 {

namespace {

// [position][channel] LDS tile.  Readers take, per 8 lanes, either 8 consecutive positions
// (q, k, bias: natural order, so that their stores walk consecutive rows) or the positions
// {x..x+3, x+16..x+19} (v: rowperm16 order).  The key (pos ^ (pos >> 2)) & 7 is distinct
// within 8 lanes for both patterns.
template <int NCH>
__device__ __forceinline__ int proj_slot(int pos, int chunk) {
  const int key = (pos ^ (pos >> 2)) & 7 & (NCH - 1);
  return pos * NCH + (chunk ^ key);
}

template <int C, int D, int NW, bool RAGGED>
__global__ __launch_bounds__(64 * NW) void triattn_proj_kernel(TriattnProjArgs p, int full_per_row, int tail_shift,
                                                               int tiles_per_batch, int total_tiles) {
  constexpr int H = 4;
  constexpr int HD = H * D;
  constexpr int NCH = C / 8;
  constexpr int LPP = NCH;
  constexpr int PPI = 64 / LPP;
  constexpr int TP = 128;
  constexpr int LN_ITERS = (TP / NW) / PPI;
  constexpr int KS = C / 16;
  constexpr int NT = HD / 32;          // 32-row output tiles per matrix (4 or 2)
  constexpr bool WIDE = (NT == 4);
  constexpr bool W16 = (NW == 16);
  // WIDE (H*D = 128), 8 waves: waves 0..3 own output tile w of q and of k, waves 4..7 own tile
  //   w-4 of v plus the bias of position tile w-4; waves w and w+4 share a SIMD, so every SIMD
  //   carries the same MFMA load.
  // WIDE, 16 waves (four per SIMD at 128 registers): waves 0..3 own tile w of q, 4..7 of k, 8..11
  //   of v, 12..15 the bias of position tile w-12; waves w, w+4, w+8, w+12 share a SIMD.
  // else (H*D = 64): waves 0..5 own one (matrix, tile) job, waves 6 and 7 do the bias of two
  //   position tiles each.
  static_assert(!W16 || WIDE, "the sixteen-wave form is built for H*D = 128");
  constexpr int TPW = 4;               // every wave visits all four position tiles
  static_assert(NT == 4 || NT == 2, "H*D must be 128 or 64");

  __shared__ u32x4_t tile[2][TP * NCH];
  __shared__ u32x4_t wb_lds[KS * 64];  // triangle-bias weights in MFMA A-operand order (rows >= H are zero)

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63, l32 = lane & 31, lh = lane >> 5;
  const int ln_chunk = lane % LPP, ln_pp = lane / LPP;

  float lw[8], lb[8];
  load_affine8(p.ln_w, ln_chunk, lw);
  load_affine8(p.ln_b, ln_chunk, lb);

  if (wave == 0) {
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      u32x4_t w = {0u, 0u, 0u, 0u};
      if (l32 < H) w = *reinterpret_cast<const u32x4_t*>(p.w_b + l32 * C + 16 * s + 8 * lh);
      wb_lds[s * 64 + lane] = w;
    }
  }  // published by the first tile's barrier
  const float qscale = kLog2e * __builtin_amdgcn_rsqf((float)D);

  const int N = p.N, Jp = p.Jp;
  // tile -> batch element, first row, first column, log2 of the width (wave-uniform); the last ragged piece
  // is moved up to end at the last row, so every row of a tile exists (the launcher makes sure that N >= 4)
  auto tile_origin = [&](int tile_id, int& b, int& i0, int& j0, int& shift) {
    const TilePlace t = tile_place<RAGGED>(tile_id, N, full_per_row, tail_shift, tiles_per_batch, true);
    b = t.b, i0 = t.i0, j0 = t.j0, shift = t.shift;
  };

  u32x4_t raw[LN_ITERS];
  float mraw[LN_ITERS];  // mask of the same positions (used by the lane with ln_chunk == 0)
  auto load_tile = [&](int tile_id) {
    int b, i0, j0, shift_rt;
    tile_origin(tile_id, b, i0, j0, shift_rt);
    const int shift = RAGGED ? shift_rt : 7, jmask = (1 << shift) - 1;
    const bf16_t* xrow = p.x + b * p.x_view.stride_b + i0 * p.x_view.stride_r;  // the tile's first row
    const float* mrow = p.mask ? p.mask + b * p.mask_view.stride_b + i0 * p.mask_view.stride_r : nullptr;
#pragma unroll
    for (int it = 0; it < LN_ITERS; ++it) {
      const int pos = wave * (TP / NW) + it * PPI + ln_pp;
      const int di = RAGGED ? pos >> shift : 0, j = j0 + (RAGGED ? pos & jmask : pos);  // every row i0 + di exists
      u32x4_t v = {0u, 0u, 0u, 0u};
      float m = 1.f;
      if (j < N) {
        v = *reinterpret_cast<const u32x4_t*>(xrow + di * p.x_view.stride_r + j * p.x_view.stride_k + 8 * ln_chunk);
        if (mrow && ln_chunk == 0) m = mrow[di * p.mask_view.stride_r + j * p.mask_view.stride_k];
      }
      raw[it] = v;
      mraw[it] = m;
    }
  };

  // Every job takes the positions in natural order: position 32*tt + l32 is column l32 of
  // position tile tt (q, k, bias: activations are the MFMA B operand) or, for v, row
  // rowperm16(l32) of it (activations are the A operand, so that a lane ends up with 16
  // consecutive keys of one channel: 32 contiguous bytes of the V^T panel).
  const int krow = rowperm16(l32);

  // A wave's role is fixed for the kernel, and each role runs its own copy of the tile loop:
  //   role 0  q and k of output tile w (H*D = 128), or one of them (H*D = 64: waves 0..3)
  //   role 1  v of output tile w-4 plus the bias of position tile w-4 (H*D = 128), or v alone
  //   role 2  bias of two position tiles (H*D = 64: waves 6, 7)
  // Inside a role every tile issues the same sequence of loads and stores.  Together with the
  // peeled first tile this lets the wait for the values loaded one tile ahead leave the
  // previous tile's stores in flight (the compiler counts them; it cannot when the number
  // depends on a branch).
  auto run = [&](auto role_tag) {
    constexpr int ROLE = decltype(role_tag)::value;
    constexpr int NJ = (ROLE == 0 && WIDE && !W16) ? 2 : (ROLE == 2 ? 0 : 1);
    const int ot = WIDE ? wave % 4 : wave % 2;
    const int m0 = ROLE == 1 ? 2 : (WIDE ? (W16 ? wave / 4 : 0) : wave / 2);  // matrix of job 0: 0 q, 1 k, 2 v

    u32x4_t wj[NJ > 0 ? NJ : 1][KS];
#pragma unroll
    for (int jj = 0; jj < NJ; ++jj) {
      const int m = m0 + jj;
      const bf16_t* W = (m == 0) ? p.w_q : (m == 1 ? p.w_k : p.w_v);
      // q, k (A operands): lane owns 16 consecutive channels (rowperm16); v (B operand): natural rows
      const int row = 32 * ot + ((ROLE == 1) ? l32 : rowperm16(l32));
#pragma unroll
      for (int s = 0; s < KS; ++s) wj[jj][s] = *reinterpret_cast<const u32x4_t*>(W + row * C + 16 * s + 8 * lh);
    }

    auto do_tile = [&](int tile_id, int buf) {
      int b, i0, j0, shift_rt;
      tile_origin(tile_id, b, i0, j0, shift_rt);
      const int shift = RAGGED ? shift_rt : 7, jmask = (1 << shift) - 1;
      // row and first column of the 32-position tile tt (wave-uniform): one row, one 32-key panel
      auto tile_row = [&](int tt) { return RAGGED ? i0 + ((32 * tt) >> shift) : i0; };
      auto tile_col = [&](int tt) { return RAGGED ? j0 + ((32 * tt) & jmask) : j0 + 32 * tt; };

      // ---- LayerNorm phase (+ mask bias, one lane per position)
#pragma unroll
      for (int it = 0; it < LN_ITERS; ++it) {
        const int pos = wave * (TP / NW) + it * PPI + ln_pp;
        tile[buf][proj_slot<NCH>(pos, ln_chunk)] = layer_norm_chunk<C>(raw[it], lw, lb);
        if (ln_chunk == 0) {
          const int i = RAGGED ? i0 + (pos >> shift) : i0, j = j0 + (RAGGED ? pos & jmask : pos);
          float mb = -__builtin_inff();
          if (j < N) mb = kLog2e * (p.inf * (mraw[it] - 1.f));
          p.mbias[((size_t)b * N + i) * Jp + j] = mb;
        }
      }
      if (tile_id + (int)gridDim.x < total_tiles) load_tile(tile_id + gridDim.x);
      __syncthreads();  // the only barrier per tile (the LDS tile is double buffered)

      // ---- projection phase
      auto bias_tile = [&](int tt) {  // triangle bias of position tile tt (wave-uniform, may be a run-time value)
        const int pos = 32 * tt + l32, i = tile_row(tt), j = tile_col(tt) + l32;
        f32x16_t acc = zero16();
#pragma unroll
        for (int s = 0; s < KS; ++s)
          acc = mfma_32x32x16(wb_lds[s * 64 + lane], tile[buf][proj_slot<NCH>(pos, 2 * s + lh)], acc);
        // rows 0..3 of the result sit in registers 0..3 of lanes 0..31
        if (lh == 0) {
#pragma unroll
          for (int h = 0; h < H; ++h) p.tbias[(((size_t)b * H + h) * N + i) * Jp + j] = (j < N) ? acc[h] * kLog2e : 0.f;
        }
      };
      if (ROLE == 2) {
        if (W16) {
          bias_tile(wave - 12);
        } else {
          bias_tile(2 * (wave - 6));
          bias_tile(2 * (wave - 6) + 1);
        }
        return;
      }
#pragma unroll
      for (int tt = 0; tt < TPW; ++tt) {
        const size_t bi = (size_t)b * N + tile_row(tt);
        const int jt = tile_col(tt);
#pragma unroll
        for (int jj = 0; jj < NJ; ++jj) {
          f32x16_t acc = zero16();
          u32x4_t o0, o1;
          bf16_t* dst;
          if (ROLE == 1) {
            // V^T panel of this position tile: rows = keys (A), columns = channels (B)
            const int kpos = 32 * tt + krow;
#pragma unroll
            for (int s = 0; s < KS; ++s)
              acc = mfma_32x32x16(tile[buf][proj_slot<NCH>(kpos, 2 * s + lh)], wj[jj][s], acc);
            // lane: channel 32*ot + l32 = head*D + d, keys 16*lh + (0..15) of the panel
            const int ch = 32 * ot + l32;
            const int head = ch / D, d = ch % D;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              o0[q] = pack_bf16(acc[2 * q], acc[2 * q + 1]);
              o1[q] = pack_bf16(acc[8 + 2 * q], acc[8 + 2 * q + 1]);
            }
            dst = p.vt + (bi * H + head) * D * Jp + (size_t)(jt >> 5) * (D * 32) + d * 32 + 16 * lh;
          } else {
            // the activation operand is re-read from LDS by every job: cheaper than holding it in
            // 32 registers across the jobs
            const int pos = 32 * tt + l32;
#pragma unroll
            for (int s = 0; s < KS; ++s)
              acc = mfma_32x32x16(wj[jj][s], tile[buf][proj_slot<NCH>(pos, 2 * s + lh)], acc);
            // lane owns channels 32*ot + 16*lh + v  ->  head, d0 .. d0+15
            const int ch0 = 32 * ot + 16 * lh;
            const int head = ch0 / D, d0 = ch0 % D;
            const bool is_q = (m0 + jj) == 0;
            const float sc = is_q ? qscale : 1.f;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              o0[q] = pack_bf16(acc[2 * q] * sc, acc[2 * q + 1] * sc);
              o1[q] = pack_bf16(acc[8 + 2 * q] * sc, acc[8 + 2 * q + 1] * sc);
            }
            dst = (is_q ? p.q : p.k) + ((bi * H + head) * Jp + jt + l32) * D + d0;
          }
          *reinterpret_cast<u32x4_t*>(dst) = o0;
          *reinterpret_cast<u32x4_t*>(dst + 8) = o1;
        }
      }
      if (ROLE == 1 && WIDE && !W16) bias_tile(wave - 4);
    };

    int tile_id = blockIdx.x;
    int buf = 0;
    if (tile_id < total_tiles) {
      load_tile(tile_id);
      do_tile(tile_id, buf);
      tile_id += gridDim.x;
      buf ^= 1;
    }
    for (; tile_id < total_tiles; tile_id += gridDim.x, buf ^= 1) do_tile(tile_id, buf);
  };

  if (W16) {
    if (wave < 8) run(std::integral_constant<int, 0>{});
    else if (wave < 12) run(std::integral_constant<int, 1>{});
    else run(std::integral_constant<int, 2>{});
  } else if (WIDE) {
    if (wave < 4) run(std::integral_constant<int, 0>{});
    else run(std::integral_constant<int, 1>{});
  } else {
    if (wave < 4) run(std::integral_constant<int, 0>{});
    else if (wave < 6) run(std::integral_constant<int, 1>{});
    else run(std::integral_constant<int, 2>{});
  }
}

template <int C, int D, int NW, bool RAGGED>
hipError_t launch(const TriattnProjArgs& a, hipStream_t stream) {
  auto kern = triattn_proj_kernel<C, D, NW, RAGGED>;
  static int cache[kMaxDevices];
  int grid_cap = 0;
  hipError_t e = per_device(cache, [&](int dev, int* v) { return resident_blocks(kern, 64 * NW, dev, v); }, &grid_cap);
  if (e != hipSuccess) return e;
  RaggedTiles t = {a.Jp / 128, 7, a.N * (a.Jp / 128)};  // whole (padded) rows in 128-wide pieces
  if (RAGGED) t = ragged_tiles(a.N, 5);                 // pieces of whole 32-key panels
  const long total = (long)a.B * t.per_batch;
  if (total > 0x7fffffffL) return hipErrorInvalidValue;
  const int grid = (int)(total < grid_cap ? total : grid_cap);
  hipLaunchKernelGGL(kern, dim3(grid), dim3(64 * NW), 0, stream, a, t.full_per_row, t.tail_shift, t.per_batch, (int)total);
  return hipGetLastError();
}

}  // namespace

hipError_t triattn_proj_launch(const TriattnProjArgs& args, int C, int D, hipStream_t stream) {
  if (args.H != 4) return hipErrorInvalidValue;
  // ragged pieces hold up to four rows, all of which must exist
  const bool ragged = args.N % 128 != 0 && args.N >= 4;
  if (C == 128 && D == 32) return ragged ? launch<128, 32, OF3_TP_WAVES, true>(args, stream) : launch<128, 32, OF3_TP_WAVES, false>(args, stream);
  if (C == 64 && D == 16) return ragged ? launch<64, 16, 8, true>(args, stream) : launch<64, 16, 8, false>(args, stream);
  return hipErrorInvalidValue;
}

}  // namespace of3

// Triangle-multiplication input pass: LayerNorm(z) and the four gated projections
//     a = mask * sigmoid(zn Wag^T) * (zn Wap^T),   b = mask * sigmoid(zn Wbg^T) * (zn Wbp^T)
// (triangular_multiplicative_update.py:485-493), written channel-major in the k-panel
// layout a[b][c][k/32][r][k%32] the contraction kernel streams from, so that the
// contraction is a plain "row times row" product for both directions: the caller's PairView
// makes (r, k) = (i, k) for the outgoing update and (r, k) = (i, k) of the transposed tensor
// for the incoming one.
//
// HBM bound (reads z once, writes a and b once).  Persistent work-groups of 8 waves (two
// per SIMD, so one wave's MFMAs overlap the other's VALU work) keep the four weight
// matrices in registers as MFMA A operands, one 32-row slice pair per wave; each tile of
// 128 positions is normalised in registers (statistics by DPP lane permutations), staged
// once in LDS as bf16 and consumed as the MFMA B operand by all waves.  The LDS tile is
// double buffered, which leaves a single barrier per tile.  Positions are dealt to MFMA
// columns so that a lane finishes 4 consecutive k of one row and channel and stores them as
// one 8-byte vector.  A tile is 4 consecutive rows r of one 32-wide k-panel: in the k-panel
// layout these are 256 contiguous bytes per channel, so 32 lanes write whole 128-byte lines.
// Only the panels that hold a k below N are written (the last one with zeros from N on), and only
// the rows up to N rounded up to 4: the contraction sums over no other panel, and what it makes of
// the other rows lands in rows and columns of x that nobody reads.
#include "of3_device.h"
#include "of3_kernels.h"
#include "of3_launch.h"

namespace of3 {

namespace {

template <int C, int CH>
__global__ __launch_bounds__(512) void trimul_proj_kernel(TrimulProjArgs p, int panels, int total_tiles) {
  constexpr int NCH = C / 8;        // 16-byte chunks per position
  constexpr int LPP = NCH;          // lanes sharing one position in the LayerNorm phase
  constexpr int PPI = 64 / LPP;     // positions per wave instruction
  constexpr int TP = 128;           // positions per tile: TR rows x one 32-wide k-panel
  constexpr int TR = TP / 32;
  constexpr int NW = 8;             // waves per work-group (two per SIMD)
  constexpr int LN_ITERS = (TP / NW) / PPI;
  constexpr int KS = C / 16;        // MFMA k-steps
  constexpr int OT = CH / 32;       // 32-row output tiles per matrix
  constexpr int NJOBS = 2 * OT;     // (a|b, output tile) jobs: 8 or 4
  constexpr int WPJ = NW / NJOBS;   // waves sharing a job: 1 or 2, each takes 4/WPJ position tiles
  constexpr int TPW = 4 / WPJ;      // position tiles per wave: 4 or 2
  constexpr int KSH = (TPW == 4) ? 2 : 1;  // swizzle key from pos / TPW: distinct for the 8 lanes of a read group
  static_assert(NJOBS == 8 || NJOBS == 4, "CH must be 128 or 64");

  // two tiles: LayerNorm of tile n+1 is written while other waves still read tile n
  __shared__ u32x4_t tile[2][TP * NCH];

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63, l32 = lane & 31, lh = lane >> 5;
  const int ln_chunk = lane % LPP, ln_pp = lane / LPP;

  // LayerNorm affine parameters of this lane's 8 channels, kept packed (8 registers instead
  // of 16) and unpacked once per tile
  u32x4_t lw_pk = *reinterpret_cast<const u32x4_t*>(p.ln_w + 8 * ln_chunk);
  u32x4_t lb_pk = *reinterpret_cast<const u32x4_t*>(p.ln_b + 8 * ln_chunk);
  __asm__ volatile("" : "+v"(lw_pk), "+v"(lb_pk));  // waited for here, once

  // this wave's job: gate and projection rows 32*ot .. +31 of a (pair 0) or b (pair 1),
  // resident in registers as MFMA A operands for the whole kernel
  const int job = wave % NJOBS, tgroup = wave / NJOBS;
  const int pair = job / OT, ot = job % OT;
  u32x4_t wg[KS], wp[KS];
  {
    const bf16_t* Wg = pair ? p.w_bg : p.w_ag;
    const bf16_t* Wp = pair ? p.w_bp : p.w_ap;
    const int row = 32 * ot + l32;
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      wg[s] = *reinterpret_cast<const u32x4_t*>(Wg + row * C + 16 * s + 8 * lh);
      wp[s] = *reinterpret_cast<const u32x4_t*>(Wp + row * C + 16 * s + 8 * lh);
    }
    // the weights count as used here: the compiler waits for them once, before the tile loop,
    // instead of carrying "may still be in flight" into every iteration (where its wait for
    // them would also be a wait for the tile's prefetch and the previous tile's stores)
#pragma unroll
    for (int s = 0; s < KS; ++s) __asm__ volatile("" : "+v"(wg[s]), "+v"(wp[s]));
  }
  bf16_t* const out = pair ? p.b : p.a;

  const int N = p.N, Np = p.Np;
  const int tiles_per_batch = ((N + TR - 1) / TR) * panels;

  // LayerNorm-phase positions of this lane: wave w takes positions [16w, 16w+16) of the tile,
  // i.e. 16 consecutive k of row w/2; iteration `it` adds PPI positions.  The lane-dependent
  // part of the address is computed once, the tile adds a wave-uniform base.
  const int ln_pos0 = wave * (TP / NW) + ln_pp;
  const int ln_row = ln_pos0 >> 5, ln_k = ln_pos0 & 31;
  // Everything a tile reads from global memory (its z values and this lane's mask values) is
  // requested one tile ahead by a fixed number of unconditional loads (positions past the end
  // are clamped to the last one and zeroed through the mask value), and every tile issues the
  // same 16 stores (the padding rows of a and b are written too, with zeros).  With fixed
  // counts the compiler's wait for the prefetched values can leave the previous tile's stores
  // in flight; with a load or store under a condition it cannot, and waits for all of them.
  u32x4_t raw[LN_ITERS];
  float mraw[TPW];
  const float* const mask_base = p.mask ? p.mask : reinterpret_cast<const float*>(p.ln_w);  // dummy when absent
  const int64_t msb = p.mask ? p.mask_view.stride_b : 0, msr = p.mask ? p.mask_view.stride_r : 0,
                msk = p.mask ? p.mask_view.stride_k : 0;
  // Positions of the tile are dealt to MFMA columns so that a lane finishes TPW consecutive
  // positions: position  32*TPW*tgroup + TPW*l32 + tt  is column l32 of this wave's tile tt.
  const int pos0 = 32 * TPW * tgroup + TPW * l32;
  auto load_tile = [&](int tile_id) {
    const int b = tile_id / tiles_per_batch;
    const int rem = tile_id - b * tiles_per_batch;
    const int r0 = (rem / panels) * TR;
    const int k0 = (rem % panels) * 32;
    int row = r0 + ln_row;
    row = row < N ? row : N - 1;
    const bf16_t* base = p.z + b * p.z_view.stride_b + row * p.z_view.stride_r + 8 * ln_chunk;
#pragma unroll
    for (int it = 0; it < LN_ITERS; ++it) {
      int k = k0 + ln_k + it * PPI;
      k = k < N ? k : N - 1;
      raw[it] = *reinterpret_cast<const u32x4_t*>(base + k * p.z_view.stride_k);
    }
    int mr = r0 + (pos0 >> 5);
    mr = mr < N ? mr : N - 1;
    const float* mrow = mask_base + b * msb + mr * msr;
#pragma unroll
    for (int tt = 0; tt < TPW; ++tt) {
      int k = k0 + (pos0 & 31) + tt;
      k = k < N ? k : N - 1;
      mraw[tt] = mrow[k * msk];
    }
  };

  auto do_tile = [&](int tile_id, int buf) {
    const int b = tile_id / tiles_per_batch;
    const int rem = tile_id - b * tiles_per_batch;
    const int r = (rem / panels) * TR + (pos0 >> 5);  // this lane's row and first k
    const int kfirst = (rem % panels) * 32 + (pos0 & 31);

    float mval[TPW];
#pragma unroll
    for (int tt = 0; tt < TPW; ++tt) mval[tt] = (kfirst + tt < N && r < N) ? (p.mask ? mraw[tt] : 1.f) : 0.f;
    bool not_one = false;
#pragma unroll
    for (int tt = 0; tt < TPW; ++tt) not_one |= mval[tt] != 1.f;
    const bool masked = __builtin_amdgcn_ballot_w64(not_one) != 0;  // wave-uniform

    // ---- LayerNorm phase: wave w normalises positions [16w, 16w+16) of the tile
    float lw[8], lb[8];
    {
      u32x4_t tw = lw_pk, tb = lb_pk;
      __asm__ volatile("" : "+v"(tw), "+v"(tb));  // keeps the unpacked copies from being hoisted out of the loop
      unpack8(tw, lw);
      unpack8(tb, lb);
    }
#pragma unroll
    for (int it = 0; it < LN_ITERS; ++it) {
      const int pos = wave * (TP / NW) + it * PPI + ln_pp;
      tile[buf][tile_slot<NCH, KSH>(pos, ln_chunk)] = layer_norm_chunk<C>(raw[it], lw, lb);
    }
    // next tile's z travels while this tile's matrix phase runs
    if (tile_id + (int)gridDim.x < total_tiles) load_tile(tile_id + gridDim.x);
    // One barrier per tile: it publishes this tile, and since every wave has finished the
    // previous tile's matrix phase before arriving, the other buffer may be overwritten by
    // the next LayerNorm phase.
    __syncthreads();

    // ---- projection phase
    float res[TPW][16];
#pragma unroll
    for (int tt = 0; tt < TPW; ++tt) {
      f32x16_t accg = zero16(), accp = zero16();
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        const u32x4_t bop = tile[buf][tile_slot<NCH, KSH>(pos0 + tt, 2 * s + lh)];
        accg = mfma_32x32x16(wg[s], bop, accg);
        accp = mfma_32x32x16(wp[s], bop, accp);
      }
      // mask * sigmoid(gate) * projection; a wave whose positions all carry mask 1 (the usual tile)
      // skips the multiplication by 1
      if (masked) {
#pragma unroll
        for (int v = 0; v < 16; ++v) res[tt][v] = (mval[tt] * sigmoidf_fast(accg[v])) * accp[v];
      } else {
#pragma unroll
        for (int v = 0; v < 16; ++v) res[tt][v] = sigmoidf_fast(accg[v]) * accp[v];
      }
    }
    // stores: register v of a lane is channel 32*ot + 8*(v/4) + 4*lh + v%4; k-panel layout
    // plane[k / 32][row][k % 32].  r < Np always (Np is a multiple of 128): rows between N and
    // Np receive zeros
    {
      // lane base: channel 32*ot + 4*lh of this batch element, row r, first k of the lane;
      // the 16 registers add wave-uniform channel offsets
      const size_t plane = (size_t)Np * Np;
      bf16_t* dst0 = out + ((size_t)b * CH + 32 * ot + 4 * lh) * plane + (size_t)(kfirst >> 5) * (Np * 32) + r * 32 +
                     (kfirst & 31);
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        bf16_t* dst = dst0 + (size_t)(8 * (v >> 2) + (v & 3)) * plane;
        if (TPW == 4) {
          u32x2_t w2 = {pack_bf16(res[0][v], res[1][v]), pack_bf16(res[2][v], res[3][v])};
          *reinterpret_cast<u32x2_t*>(dst) = w2;
        } else {
          *reinterpret_cast<uint32_t*>(dst) = pack_bf16(res[0][v], res[1][v]);
        }
      }
    }
  };

  // the first tile is peeled: the loop proper is only entered with a tile's stores in flight
  int tile_id = blockIdx.x;
  int buf = 0;
  if (tile_id < total_tiles) {
    load_tile(tile_id);
    do_tile(tile_id, buf);
    tile_id += gridDim.x;
    buf ^= 1;
  }
  for (; tile_id < total_tiles; tile_id += gridDim.x, buf ^= 1) do_tile(tile_id, buf);
}

template <int C, int CH>
hipError_t launch(const TrimulProjArgs& a, hipStream_t stream) {
  auto kern = trimul_proj_kernel<C, CH>;
  static int cache[kMaxDevices];
  int grid_cap = 0;
  hipError_t e = per_device(cache, [&](int dev, int* v) { return resident_blocks(kern, 512, dev, v); }, &grid_cap);
  if (e != hipSuccess) return e;
  const int panels = (a.N + 31) / 32;  // the panels that hold a k below N; the contraction reads no others
  const long total = (long)a.B * ((a.N + 3) / 4) * panels;
  const int grid = (int)(total < grid_cap ? total : grid_cap);
  hipLaunchKernelGGL(kern, dim3(grid), dim3(512), 0, stream, a, panels, (int)total);
  return hipGetLastError();
}

}  // namespace

hipError_t trimul_proj_launch(const TrimulProjArgs& args, int C, int CH, hipStream_t stream) {
  if (C == 128 && CH == 128) return launch<128, 128>(args, stream);
  if (C == 64 && CH == 64) return launch<64, 64>(args, stream);
  return hipErrorInvalidValue;
}

}  // namespace of3

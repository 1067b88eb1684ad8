// Triangle-multiplication input pass: LayerNorm(z) and the four gated projections
//     a = mask * sigmoid(zn Wag^T) * (zn Wap^T),   b = mask * sigmoid(zn Wbg^T) * (zn Wbp^T)
// (triangular_multiplicative_update.py:485-493), written channel-major in the k-panel
// layout a[b][c][k/32][r][k%32] the contraction kernel streams from, so that the
// contraction is a plain "row times row" product for both directions: the caller's PairView
// makes (r, k) = (i, k) for the outgoing update and (r, k) = (i, k) of the transposed tensor
// for the incoming one.
//
// HBM bound (reads z once, writes a and b once).  Persistent work-groups keep their slice
// of the four weight matrices in registers as MFMA A operands; each tile of 128
// positions is normalised in registers, staged once in LDS as bf16 and consumed as the
// MFMA B operand by all four waves.  Position 4*l+t of the tile sits in column l of
// position-tile t, so after four tiles a lane owns 4 consecutive positions of a channel
// and stores them as one 8-byte vector (8 lanes fill one 64-byte panel row).
#include "of3_device.h"
#include "of3_kernels.h"

namespace of3 {

namespace {

template <int C, int CH>
__global__ __launch_bounds__(256) void trimul_proj_kernel(TrimulProjArgs p, int tiles_per_row, int total_tiles) {
  constexpr int NCH = C / 8;        // 16-byte chunks per position
  constexpr int LPP = NCH;          // lanes sharing one position in the LayerNorm phase
  constexpr int PPI = 64 / LPP;     // positions per wave instruction
  constexpr int TP = 128;           // positions per tile
  constexpr int LN_ITERS = 32 / PPI;
  constexpr int KS = C / 16;        // MFMA k-steps
  constexpr int OT = CH / 32;       // 32-row output tiles per matrix
  constexpr int NJ = (2 * OT) / 4;  // (matrix pair, output tile) jobs per wave
  static_assert(NJ >= 1, "CH must be at least 64");

  __shared__ u32x4_t tile[TP * NCH];

  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63, l32 = lane & 31, lh = lane >> 5;
  const int ln_chunk = lane % LPP, ln_pp = lane / LPP;

  float lw[8], lb[8];
  load_affine8(p.ln_w, ln_chunk, lw);
  load_affine8(p.ln_b, ln_chunk, lb);

  // weights of this wave's jobs, resident for the whole kernel
  u32x4_t wg[NJ][KS], wp[NJ][KS];
#pragma unroll
  for (int jj = 0; jj < NJ; ++jj) {
    const int idx = wave * NJ + jj;
    const int pair = idx / OT, ot = idx % OT;
    const bf16_t* Wg = pair ? p.w_bg : p.w_ag;
    const bf16_t* Wp = pair ? p.w_bp : p.w_ap;
    const int row = 32 * ot + l32;
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      wg[jj][s] = *reinterpret_cast<const u32x4_t*>(Wg + row * C + 16 * s + 8 * lh);
      wp[jj][s] = *reinterpret_cast<const u32x4_t*>(Wp + row * C + 16 * s + 8 * lh);
    }
  }

  const int N = p.N, Np = p.Np;
  const int tiles_per_batch = N * tiles_per_row;

  u32x4_t raw[LN_ITERS];
  auto load_tile = [&](int tile_id) {
    const int b = tile_id / tiles_per_batch;
    const int rem = tile_id - b * tiles_per_batch;
    const int r = rem / tiles_per_row;
    const int k0 = (rem - r * tiles_per_row) * TP;
    const bf16_t* zrow = p.z + b * p.z_view.stride_b + r * p.z_view.stride_r;
#pragma unroll
    for (int it = 0; it < LN_ITERS; ++it) {
      const int k = k0 + wave * 32 + it * PPI + ln_pp;
      u32x4_t v = {0u, 0u, 0u, 0u};
      if (k < N) v = *reinterpret_cast<const u32x4_t*>(zrow + k * p.z_view.stride_k + 8 * ln_chunk);
      raw[it] = v;
    }
  };

  int tile_id = blockIdx.x;
  if (tile_id < total_tiles) load_tile(tile_id);

  for (; tile_id < total_tiles; tile_id += gridDim.x) {
    const int b = tile_id / tiles_per_batch;
    const int rem = tile_id - b * tiles_per_batch;
    const int r = rem / tiles_per_row;
    const int k0 = (rem - r * tiles_per_row) * TP;

    // mask of the 4 positions this lane finishes: tile positions 4*l32 + t
    float mval[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const int k = k0 + 4 * l32 + t;
      float m = 0.f;
      if (k < N) {
        m = 1.f;
        if (p.mask) m = p.mask[b * p.mask_view.stride_b + r * p.mask_view.stride_r + k * p.mask_view.stride_k];
      }
      mval[t] = m;
    }

    // ---- LayerNorm phase: wave w normalises positions [32w, 32w+32) of the tile
#pragma unroll
    for (int it = 0; it < LN_ITERS; ++it) {
      const int pos = wave * 32 + it * PPI + ln_pp;
      tile[tile_slot<NCH, 2>(pos, ln_chunk)] = layer_norm_chunk<C>(raw[it], lw, lb);
    }
    __syncthreads();

    // prefetch the next tile while the matrix phase runs
    if (tile_id + (int)gridDim.x < total_tiles) load_tile(tile_id + gridDim.x);

    // ---- projection phase, one (matrix pair, output tile) job at a time
#pragma unroll
    for (int jj = 0; jj < NJ; ++jj) {
      uint32_t pk[2][16];
      float prev[16];
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const int pos = 4 * l32 + t;
        f32x16_t accg = zero16(), accp = zero16();
#pragma unroll
        for (int s = 0; s < KS; ++s) {
          const u32x4_t bop = tile[tile_slot<NCH, 2>(pos, 2 * s + lh)];
          accg = mfma_32x32x16(wg[jj][s], bop, accg);
          accp = mfma_32x32x16(wp[jj][s], bop, accp);
        }
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const float val = (mval[t] * sigmoidf_fast(accg[v])) * accp[v];
          if (t & 1)
            pk[t >> 1][v] = pack_bf16(prev[v], val);
          else
            prev[v] = val;
        }
      }
      // stores: register v of a lane is channel 32*ot + 8*(v/4) + 4*lh + v%4
      const int idx = wave * NJ + jj;
      const int pair = idx / OT, ot = idx % OT;
      bf16_t* out = pair ? p.b : p.a;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int ch = 32 * ot + 8 * (v >> 2) + 4 * lh + (v & 3);
        // k-panel layout: plane[k / 32][row][k % 32]
        const int k = k0 + 4 * l32;
        bf16_t* dst = out + ((size_t)b * CH + ch) * Np * Np + (size_t)(k >> 5) * (Np * 32) + r * 32 + (k & 31);
        u32x2_t w2 = {pk[0][v], pk[1][v]};
        *reinterpret_cast<u32x2_t*>(dst) = w2;
      }
    }
    __syncthreads();  // tile[] is rewritten by the next iteration
  }
}

template <int C, int CH>
hipError_t launch(const TrimulProjArgs& a, hipStream_t stream) {
  auto kern = trimul_proj_kernel<C, CH>;
  static int grid_cap = 0;
  if (grid_cap == 0) {
    int dev = 0, cus = 0, per_cu = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    if (e != hipSuccess) return e;
    e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kern, 256, 0);
    if (e != hipSuccess) return e;
    grid_cap = cus * (per_cu > 0 ? per_cu : 1);
  }
  const int tiles_per_row = a.Np / 128;
  const long total = (long)a.B * a.N * tiles_per_row;
  const int grid = (int)(total < grid_cap ? total : grid_cap);
  hipLaunchKernelGGL(kern, dim3(grid), dim3(256), 0, stream, a, tiles_per_row, (int)total);
  return hipGetLastError();
}

}  // namespace

hipError_t trimul_proj_launch(const TrimulProjArgs& args, int C, int CH, hipStream_t stream) {
  if (C == 128 && CH == 128) return launch<128, 128>(args, stream);
  if (C == 64 && CH == 64) return launch<64, 64>(args, stream);
  return hipErrorInvalidValue;
}

}  // namespace of3

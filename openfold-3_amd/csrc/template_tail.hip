// End of the template branch (template_module.py):
//   * TemplatePairStack's closing LayerNorm over c_t (:376, normalization.py:65-84),
//   * the tail of TemplateEmbedderAllAtom.forward (:462-465):
//         out[b, i, j, :] = W_t . relu( (1/T) sum_t LN(t[b, t, i, j, :]) )        (linear_t has no bias)
// Both are position-wise and HBM bound.  The fused tail reads the T template planes once and
// writes one c_z plane; nothing of size T x N x N x c_t is written in between.
//
// bf16 rounding points are the reference's: the LayerNorm output, the sum over the templates
// (torch.sum accumulates in fp32 and rounds once), the division by T, the linear output.
//
// Tail kernel: work-group = 8 independent waves, a wave owns 32 consecutive positions.
// LayerNorm in registers (a position's channels spread over c_t/8 lanes, statistics by DPP),
// the T normalised planes summed in fp32 registers, mean + ReLU written as bf16 into a
// wave-private LDS tile [position][channel]; linear_t with the weights as MFMA A operands held
// in registers (rows dealt by rowperm16: a lane ends up with 16 consecutive output channels of
// one position, 32 contiguous bytes) and the positions as B operands read from the LDS tile.
#include "of3_device.h"
#include "of3_kernels.h"
#include "of3_launch.h"

namespace of3 {

namespace {

// 16-byte chunks of a position are XOR-ed with this key; the 16 lanes of one LDS read phase hold
// 16 consecutive positions at one chunk index and must cover all 64 banks (two 128-byte rows per
// 256-byte bank window for c_t = 64)
__device__ __forceinline__ int key_c(int pos) { return (pos >> 1) & 7; }

template <int CT, int CZ>
__global__ __launch_bounds__(512) void template_tail_kernel(TemplateTailArgs p, int tiles_per_batch, int total_tiles) {
  static_assert(CT == 64, "c_t = 64: 8 lanes per position");
  constexpr int NCH = CT / 8;    // 16-byte chunks (= lanes) per position
  constexpr int PPI = 64 / NCH;  // positions per wave-wide load
  constexpr int ITERS = 32 / PPI;
  constexpr int KS = CT / 16;
  constexpr int NT = CZ / 32;

  __shared__ u32x4_t lds[8 * 32 * NCH];
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63, l32 = lane & 31, lh = lane >> 5;
  const int chunk = lane % NCH, pp = lane / NCH;
  u32x4_t* mine = lds + wave * (32 * NCH);
  const int T = p.T;
  const long P = p.P;
  const bool apply_ln = p.apply_ln != 0;

  float lw[8], lb[8];
  if (apply_ln) {
    load_affine8(p.ln_w, chunk, lw);
    load_affine8(p.ln_b, chunk, lb);
  } else {
#pragma unroll
    for (int e = 0; e < 8; ++e) lw[e] = 1.f, lb[e] = 0.f;
  }
  // A operands: output channel 32*nt + rowperm16(l32), input channels 16*s + 8*lh .. +7
  u32x4_t wreg[NT][KS];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int s = 0; s < KS; ++s)
      wreg[nt][s] = *reinterpret_cast<const u32x4_t*>(p.w + (32 * nt + rowperm16(l32)) * CT + 16 * s + 8 * lh);

  u32x4_t raw[ITERS];
  auto load_plane = [&](int tile_id, int t) {
    const int b = tile_id / tiles_per_batch;
    const long p0 = (long)(tile_id - b * tiles_per_batch) * 256 + 32 * wave;
    const bf16_t* plane = p.t + ((size_t)b * T + t) * P * CT;
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      long pos = p0 + it * PPI + pp;
      pos = pos < P ? pos : P - 1;  // positions past the end repeat the last one; they are never stored
      raw[it] = *reinterpret_cast<const u32x4_t*>(plane + pos * CT + 8 * chunk);
    }
  };
  if ((int)blockIdx.x < total_tiles) load_plane(blockIdx.x, 0);

  const float t_count = (float)T;
  for (int tile_id = blockIdx.x; tile_id < total_tiles; tile_id += gridDim.x) {
    const int b = tile_id / tiles_per_batch;
    const long p0 = (long)(tile_id - b * tiles_per_batch) * 256 + 32 * wave;

    float sum[ITERS][8];
#pragma unroll
    for (int it = 0; it < ITERS; ++it)
#pragma unroll
      for (int e = 0; e < 8; ++e) sum[it][e] = 0.f;

    for (int t = 0; t < T; ++t) {
      u32x4_t cur[ITERS];
#pragma unroll
      for (int it = 0; it < ITERS; ++it) cur[it] = raw[it];
      // the next plane of this tile, or the first plane of the next tile, is in flight meanwhile
      if (t + 1 < T) load_plane(tile_id, t + 1);
      else if (tile_id + (int)gridDim.x < total_tiles) load_plane(tile_id + gridDim.x, 0);
#pragma unroll
      for (int it = 0; it < ITERS; ++it) {
        const u32x4_t y = apply_ln ? layer_norm_chunk<CT>(cur[it], lw, lb) : cur[it];
        float f[8];
        unpack8(y, f);
#pragma unroll
        for (int e = 0; e < 8; ++e) sum[it][e] += f[e];
      }
    }

#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      const int pos = it * PPI + pp;
      float m[8];
      unpack8(pack8(sum[it]), m);  // the bf16 sum over the templates
#pragma unroll
      for (int e = 0; e < 8; ++e) m[e] = m[e] / t_count;
      unpack8(pack8(m), m);        // the bf16 mean
#pragma unroll
      for (int e = 0; e < 8; ++e) m[e] = fmaxf(m[e], 0.f);
      mine[pos * NCH + (chunk ^ key_c(pos))] = pack8(m);
    }

    u32x4_t bop[KS];
#pragma unroll
    for (int s = 0; s < KS; ++s) bop[s] = mine[l32 * NCH + ((2 * s + lh) ^ key_c(l32))];
    const long pos = p0 + l32;
    bf16_t* dst = p.out + ((size_t)b * P + (pos < P ? pos : P - 1)) * CZ + 16 * lh;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      f32x16_t acc = zero16();
#pragma unroll
      for (int s = 0; s < KS; ++s) acc = mfma_32x32x16(wreg[nt][s], bop[s], acc);
      // lane (position l32, half lh): output channels 32*nt + 16*lh + (0..15)
      if (pos < P) {
        u32x4_t o0, o1;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          o0[q] = pack_bf16(acc[2 * q], acc[2 * q + 1]);
          o1[q] = pack_bf16(acc[8 + 2 * q], acc[8 + 2 * q + 1]);
        }
        *reinterpret_cast<u32x4_t*>(dst + 32 * nt) = o0;
        *reinterpret_cast<u32x4_t*>(dst + 32 * nt + 8) = o1;
      }
    }
    // the next tile's mean overwrites the LDS tile only after this tile's operand reads have
    // returned (the MFMAs above depend on them)
  }
}

// LayerNorm over the last dimension of a contiguous [rows][C] bf16 tensor: C/8 lanes per row,
// 16 bytes per lane, four rows per lane in flight
template <int C>
__global__ __launch_bounds__(256) void layer_norm_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                                                         const bf16_t* __restrict__ b, bf16_t* __restrict__ out,
                                                         long rows) {
  constexpr int NCH = C / 8, RPI = 64 / NCH, U = 4;
  const int lane = threadIdx.x & 63, chunk = lane % NCH, rr = lane / NCH;
  float lw[8], lb[8];
  load_affine8(w, chunk, lw);
  load_affine8(b, chunk, lb);
  const long wave_id = (long)blockIdx.x * 4 + (threadIdx.x >> 6), n_waves = (long)gridDim.x * 4;
  for (long r0 = wave_id * (RPI * U); r0 < rows; r0 += n_waves * (RPI * U)) {
    u32x4_t raw[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      long r = r0 + u * RPI + rr;
      r = r < rows ? r : rows - 1;  // full groups of lanes for the DPP sums; duplicates are not stored
      raw[u] = *reinterpret_cast<const u32x4_t*>(x + r * C + 8 * chunk);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const long r = r0 + u * RPI + rr;
      const u32x4_t y = layer_norm_chunk<C>(raw[u], lw, lb);
      if (r < rows) *reinterpret_cast<u32x4_t*>(out + r * C + 8 * chunk) = y;
    }
  }
}

}  // namespace

hipError_t template_tail_launch(const TemplateTailArgs& a, int CT, int CZ, hipStream_t stream) {
  if (CT != 64 || CZ != 128 || a.T < 1 || a.P < 1 || a.B < 1) return hipErrorInvalidValue;
  auto kern = template_tail_kernel<64, 128>;
  static int cache[kMaxDevices];
  int grid_cap = 0;
  hipError_t e = per_device(cache, [&](int dev, int* v) { return resident_blocks(kern, 512, dev, v); }, &grid_cap);
  if (e != hipSuccess) return e;
  const long tiles_per_batch = (a.P + 255) / 256;
  const long total = tiles_per_batch * a.B;
  if (total > 0x7fffffffl) return hipErrorInvalidValue;
  const int grid = (int)(total < grid_cap ? total : grid_cap);
  hipLaunchKernelGGL(kern, dim3(grid), dim3(512), 0, stream, a, (int)tiles_per_batch, (int)total);
  return hipGetLastError();
}

hipError_t layer_norm_launch(const bf16_t* x, const bf16_t* w, const bf16_t* b, bf16_t* out, long rows, int C,
                             hipStream_t stream) {
  if (rows < 1 || !(C == 64 || C == 128)) return hipErrorInvalidValue;
  static int cache[kMaxDevices];
  int grid_cap = 0;
  hipError_t e = per_device(
      cache, [&](int dev, int* v) { return resident_blocks(layer_norm_kernel<128>, 256, dev, v); }, &grid_cap);
  if (e != hipSuccess) return e;
  const int rows_per_block = 4 * 4 * (64 / (C / 8));
  const long blocks = (rows + rows_per_block - 1) / rows_per_block;
  const int grid = (int)(blocks < grid_cap ? blocks : grid_cap);
  if (C == 128) hipLaunchKernelGGL(layer_norm_kernel<128>, dim3(grid), dim3(256), 0, stream, x, w, b, out, rows);
  else hipLaunchKernelGGL(layer_norm_kernel<64>, dim3(grid), dim3(256), 0, stream, x, w, b, out, rows);
  return hipGetLastError();
}

}  // namespace of3

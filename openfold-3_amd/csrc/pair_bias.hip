// Pair-bias projection of AttentionPairBias (attention_pair_bias.py:151-161, called once per
// PairFormerBlock, pairformer.py:189-201):
//     out[b][h][i][j] = sum_c LayerNorm(z[b,i,j,:])[c] * W[h][c]          (permute_final_dims [2,0,1])
// Position-wise and HBM bound: reads z once, writes H/C of its size.
//
// Work-group = 8 waves, a tile = 256 consecutive positions j of one row (b, i); a wave owns 32 of
// them and never talks to the others: LayerNorm in registers, transpose through a wave-private
// LDS tile into MFMA A operands (positions as rows), B = the H x C weights held in registers
// (lane = head, zero beyond H).  With the rows dealt by rowperm16 a lane ends up with 16
// consecutive positions of one head, i.e. 32 contiguous output bytes.
#include "of3_device.h"
#include "of3_kernels.h"
#include "of3_launch.h"

namespace of3 {

namespace {

// 16-byte chunks of a position are XOR-ed with this key; the 16 lanes of one LDS read phase hold
// positions {0..7, 16..23} or {8..15, 24..31} (rowperm16) at one chunk index and must cover all
// 64 banks: one 256-byte row per bank window (NCH = 16) or two 128-byte rows (NCH = 8)
template <int NCH>
__device__ __forceinline__ int key_p(int pos) {
  return NCH == 16 ? (pos & 7) | ((pos >> 1) & 8) : ((pos >> 1) & 3) | ((pos >> 2) & 4);
}

template <int C>
__global__ __launch_bounds__(512) void pair_bias_kernel(PairBiasArgs p, int tiles_per_row, int total_tiles) {
  constexpr int NCH = C / 8;
  constexpr int PPI = 64 / NCH;
  constexpr int ITERS = 32 / PPI;
  constexpr int KS = C / 16;

  __shared__ u32x4_t lds[8 * 32 * NCH];
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63, l32 = lane & 31, lh = lane >> 5;
  const int chunk = lane % NCH, pp = lane / NCH;
  u32x4_t* mine = lds + wave * (32 * NCH);
  const int N = p.N, H = p.H;

  float lw[8], lb[8];
  load_affine8(p.ln_w, chunk, lw);
  if (p.ln_b) {
    load_affine8(p.ln_b, chunk, lb);
  } else {
#pragma unroll
    for (int e = 0; e < 8; ++e) lb[e] = 0.f;
  }
  // B operands: head l32, channels 16*s + 8*lh .. +7
  u32x4_t wreg[KS];
#pragma unroll
  for (int s = 0; s < KS; ++s) {
    const u32x4_t zero = {0u, 0u, 0u, 0u};
    wreg[s] = l32 < H ? *reinterpret_cast<const u32x4_t*>(p.w + l32 * C + 16 * s + 8 * lh) : zero;
  }
  const int arow = rowperm16(l32);
  const int tiles_per_batch = N * tiles_per_row;
  const bool vec_ok = (N % 8) == 0;  // 16-byte aligned 16-position runs

  u32x4_t raw[ITERS];
  auto load_tile = [&](int tile_id) {
    const int b = tile_id / tiles_per_batch;
    const int rem = tile_id - b * tiles_per_batch;
    const int i = rem / tiles_per_row;
    const int j0 = (rem - i * tiles_per_row) * 256 + 32 * wave;
    const bf16_t* row = p.z + b * p.z_view.stride_b + i * p.z_view.stride_r;
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      int j = j0 + it * PPI + pp;
      j = j < N ? j : N - 1;  // positions past the end repeat the last one; they are never stored
      raw[it] = *reinterpret_cast<const u32x4_t*>(row + j * p.z_view.stride_k + 8 * chunk);
    }
  };
  if ((int)blockIdx.x < total_tiles) load_tile(blockIdx.x);

  for (int tile_id = blockIdx.x; tile_id < total_tiles; tile_id += gridDim.x) {
    const int b = tile_id / tiles_per_batch;
    const int rem = tile_id - b * tiles_per_batch;
    const int i = rem / tiles_per_row;
    const int j0 = (rem - i * tiles_per_row) * 256 + 32 * wave;

#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      const int pos = it * PPI + pp;
      mine[pos * NCH + (chunk ^ key_p<NCH>(pos))] = layer_norm_chunk<C>(raw[it], lw, lb);
    }
    if (tile_id + (int)gridDim.x < total_tiles) load_tile(tile_id + gridDim.x);

    f32x16_t acc = zero16();
#pragma unroll
    for (int s = 0; s < KS; ++s) acc = mfma_32x32x16(mine[arow * NCH + ((2 * s + lh) ^ key_p<NCH>(arow))], wreg[s], acc);

    // lane (head l32, half lh): positions j0 + 16*lh + (0..15)
    const int jl = j0 + 16 * lh;
    if (l32 < H && jl < N) {
      bf16_t* dst = p.out + (((size_t)b * H + l32) * N + i) * N + jl;
      if (vec_ok && jl + 16 <= N) {
        u32x4_t o0, o1;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          o0[q] = pack_bf16(acc[2 * q], acc[2 * q + 1]);
          o1[q] = pack_bf16(acc[8 + 2 * q], acc[8 + 2 * q + 1]);
        }
        *reinterpret_cast<u32x4_t*>(dst) = o0;
        *reinterpret_cast<u32x4_t*>(dst + 8) = o1;
      } else if (jl + 16 <= N) {
        // rows of a length that is no multiple of 8 start at any even byte: pairs of positions from the
        // first 4-byte boundary on (8 stores, or 1 + 7 + 1) instead of 16 single ones
        const bool odd = (reinterpret_cast<uintptr_t>(dst) & 2) != 0;
        if (odd) {
          dst[0] = to_bf16(acc[0]);
          dst[15] = to_bf16(acc[15]);
        }
        uint32_t* d32 = reinterpret_cast<uint32_t*>(dst + (odd ? 1 : 0));
#pragma unroll
        for (int q = 0; q < 7; ++q) d32[q] = odd ? pack_bf16(acc[2 * q + 1], acc[2 * q + 2]) : pack_bf16(acc[2 * q], acc[2 * q + 1]);
        if (!odd) d32[7] = pack_bf16(acc[14], acc[15]);
      } else {
#pragma unroll
        for (int v = 0; v < 16; ++v)
          if (jl + v < N) dst[v] = to_bf16(acc[v]);
      }
    }
    // the next tile's LayerNorm overwrites the LDS tile only after this wave's MFMA reads have
    // returned (the stores above depend on them)
  }
}

template <int C>
hipError_t launch(const PairBiasArgs& a, hipStream_t stream) {
  auto kern = pair_bias_kernel<C>;
  static int cache[kMaxDevices];
  int grid_cap = 0;
  hipError_t e = per_device(cache, [&](int dev, int* v) { return resident_blocks(kern, 512, dev, v); }, &grid_cap);
  if (e != hipSuccess) return e;
  const int tiles_per_row = (a.N + 255) / 256;
  const long total = (long)a.B * a.N * tiles_per_row;
  const int grid = (int)(total < grid_cap ? total : grid_cap);
  hipLaunchKernelGGL(kern, dim3(grid), dim3(512), 0, stream, a, tiles_per_row, (int)total);
  return hipGetLastError();
}

}  // namespace

hipError_t pair_bias_launch(const PairBiasArgs& args, int C, hipStream_t stream) {
  if (args.H < 1 || args.H > 32) return hipErrorInvalidValue;
  if (C == 128) return launch<128>(args, stream);
  if (C == 64) return launch<64>(args, stream);
  return hipErrorInvalidValue;
}

}  // namespace of3

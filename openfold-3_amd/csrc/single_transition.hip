// Transition of the single representation (SwiGLUTransition over s [*, 384], transition.py:225-271
// with activations.py:33-61; pairformer.py:203-212):
//     out = [x +] ((silu(LN(x) Wa^T) * (LN(x) Wb^T)) Wout^T) * mask,   Wa, Wb: [HID][384], Wout: [384][HID]
// Position-wise over a few thousand rows at most (5.4 GFLOP at 768 rows, n = 4): two small kernels
// built from the row tiles of the single-representation attention.
//  1. hidden: a work-group normalises 32 rows into the LDS tile; each wave computes one tile of 32
//     hidden channels for both products and writes silu(a) * b as bf16 into h [rows][HID].
//  2. out: a work-group owns 32 rows x 32 output channels, holds the rows' hidden activations in
//     LDS (one tile per slice of 384) and lets its four waves take different slices; the partial
//     tiles are added through LDS, then mask and residual.
#include "of3_device.h"
#include "of3_kernels.h"
#include "of3_launch.h"
#include "of3_rowtile.h"

namespace of3 {

namespace {

using namespace rowtile;

__global__ __launch_bounds__(256) void row_transition_hidden_kernel(RowTransitionArgs p) {
  __shared__ u32x4_t act[32 * kChunks];
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63, l32 = lane & 31, lh = lane >> 5;
  const long pos0 = (long)blockIdx.x * 32;
  fill_tile<true>(act, p.x, kK, pos0, p.rows, p.ln_w, p.ln_b, wave, lane);
  __syncthreads();
  const long pos = pos0 + l32;
  for (int tile = blockIdx.y * 4 + wave; tile < p.HID / 32; tile += gridDim.y * 4) {
    const size_t wrow = (size_t)(32 * tile + rowperm16(l32)) * kK;
    const f32x16_t a = tile_product<true>(act, p.wa + wrow, l32, lh);
    const f32x16_t b = tile_product<true>(act, p.wb + wrow, l32, lh);
    // lane (row, half lh): hidden channels 32*tile + 16*lh + v
    if (pos < p.rows) {
      u32x4_t o0, o1;
      float h[16];
#pragma unroll
      for (int v = 0; v < 16; ++v) h[v] = a[v] * sigmoidf_fast(a[v]) * b[v];
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        o0[w] = pack_bf16(h[2 * w], h[2 * w + 1]);
        o1[w] = pack_bf16(h[8 + 2 * w], h[8 + 2 * w + 1]);
      }
      bf16_t* dst = p.h + (size_t)pos * p.HID + 32 * tile + 16 * lh;
      *reinterpret_cast<u32x4_t*>(dst) = o0;
      *reinterpret_cast<u32x4_t*>(dst + 8) = o1;
    }
  }
}

// One work-group per (32 rows, 32 output channels); its waves split the hidden dimension in
// slices of 384 (wave w takes slices w, w+4, ...) and add their partial tiles through LDS.  Every
// slice of the rows' hidden activations sits in its own LDS tile, filled by all waves together.
__global__ __launch_bounds__(256) void row_transition_out_kernel(RowTransitionArgs p) {
  extern __shared__ u32x4_t dyn[];
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63, l32 = lane & 31, lh = lane >> 5;
  const long pos0 = (long)blockIdx.x * 32;
  const int tile = blockIdx.y;  // 32 output channels
  const int slices = p.HID / kK;
  u32x4_t* act = dyn;                                                  // [slices][32 * kChunks]
  float* merge = reinterpret_cast<float*>(dyn + slices * 32 * kChunks);  // [4][16][64]
  for (int sl = 0; sl < slices; ++sl)
    fill_tile<false>(act + sl * 32 * kChunks, p.h + sl * kK, p.HID, pos0, p.rows, nullptr, nullptr, wave, lane);
  __syncthreads();
  const size_t wrow = (size_t)(32 * tile + rowperm16(l32)) * p.HID;
  f32x16_t acc = zero16();
  for (int sl = wave; sl < slices; sl += 4) acc = tile_product<true>(act + sl * 32 * kChunks, p.wout + wrow + sl * kK, l32, lh, acc);
#pragma unroll
  for (int v = 0; v < 16; ++v) merge[(wave * 16 + v) * 64 + lane] = acc[v];
  __syncthreads();
  if (wave != 0) return;
#pragma unroll
  for (int w = 1; w < 4; ++w)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[v] += merge[(w * 16 + v) * 64 + lane];

  const long pos = pos0 + l32;
  if (pos < p.rows) {
    const float m = p.mask ? p.mask[pos] : 1.f;
    const size_t off = (size_t)pos * kK + 32 * tile + 16 * lh;
    float f[16];
#pragma unroll
    for (int v = 0; v < 16; ++v) f[v] = acc[v] * m;
    if (p.add_residual) {
      // the reference adds the module's bf16 output to s: round before the add
      u32x4_t r[2];
      load16_raw(p.x + off, 0, 16, true, r);
#pragma unroll
      for (int w = 0; w < 8; ++w) {
        f[2 * w] = bf16_to_f32(to_bf16(f[2 * w])) + bf16_lo(r[w >> 2][w & 3]);
        f[2 * w + 1] = bf16_to_f32(to_bf16(f[2 * w + 1])) + bf16_hi(r[w >> 2][w & 3]);
      }
    }
    u32x4_t o0, o1;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      o0[w] = pack_bf16(f[2 * w], f[2 * w + 1]);
      o1[w] = pack_bf16(f[8 + 2 * w], f[8 + 2 * w + 1]);
    }
    *reinterpret_cast<u32x4_t*>(p.out + off) = o0;
    *reinterpret_cast<u32x4_t*>(p.out + off + 8) = o1;
  }
}

}  // namespace

hipError_t row_transition_launch(const RowTransitionArgs& a, hipStream_t stream) {
  if (a.rows < 1 || a.HID < kK || (a.HID % kK) != 0) return hipErrorInvalidValue;
  const long row_blocks = (a.rows + 31) / 32;
  if (row_blocks > 0x7fffffffl) return hipErrorInvalidValue;
  const int hidden_groups = a.HID / 32 / 4;  // one hidden tile per wave
  if (hidden_groups > 65535) return hipErrorInvalidValue;
  hipLaunchKernelGGL(row_transition_hidden_kernel, dim3((unsigned)row_blocks, hidden_groups), dim3(256), 0, stream, a);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return e;
  // LDS: one tile per hidden slice plus the merge area; at most 5 slices fit a CU's 160 KB
  const int slices = a.HID / kK;
  const size_t smem = (size_t)slices * 32 * kChunks * sizeof(u32x4_t) + 4 * 16 * 64 * sizeof(float);
  if (smem > 160 * 1024) return hipErrorInvalidValue;
  static int cache[kMaxDevices];
  int configured = 0;
  e = per_device(
      cache,
      [&](int, int* v) {
        *v = 1;
        return hipFuncSetAttribute(reinterpret_cast<const void*>(row_transition_out_kernel),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
      },
      &configured);
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(row_transition_out_kernel, dim3((unsigned)row_blocks, kK / 32), dim3(256), smem, stream, a);
  return hipGetLastError();
}

}  // namespace of3

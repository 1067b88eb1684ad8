// Triangle-multiplication contraction: for every (batch, channel) plane
//     X[i][j] = sum_k A[i][k] * Bm[j][k]
// with A, Bm, X dense row-major [Np][Np] bf16 planes (Np a multiple of 128, zero-padded
// along k by the projection kernel).  This is the reference's per-channel matrix product
// of _combine_projections (triangular_multiplicative_update.py:71-97); the projection
// kernel has already laid both operands out k-contiguous for either direction, so one
// "row times row" kernel serves the outgoing and the incoming update.
//
// MFMA bound.  Work-group = 4 waves, tile BM (j) x BN (i); k is consumed 64 at a time
// through a double-buffered, XOR-swizzled LDS stage filled with coalesced 16-byte loads.
// The j side is the MFMA M side so that a lane ends up owning 16*TM consecutive j of one
// output row i and can store them as 16-byte vectors.
#include "of3_device.h"
#include "of3_kernels.h"

namespace of3 {

namespace {

constexpr int kBK = 64;  // k per stage (128 bytes per row = 8 chunks)

template <int HB>
__device__ __forceinline__ int key_m(int row) { return (row & 3) | (((row >> HB) & 1) << 2); }
__device__ __forceinline__ int key_n(int row) { return row & 7; }

template <int BM, int BN, int WAVES_M, int WAVES_N>
__global__ __launch_bounds__(256) void contract_kernel(const bf16_t* __restrict__ pm,  // j side [batch][Np][Np]
                                                       const bf16_t* __restrict__ pn,  // i side
                                                       bf16_t* __restrict__ x, int Np, int tiles_m,
                                                       int tiles_n, int total, int per_xcd) {
  static_assert(WAVES_M * WAVES_N == 4, "four waves per work-group");
  constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
  constexpr int TM = WM / 32, TN = WN / 32;
  constexpr int HB = (TM == 4) ? 6 : (TM == 2 ? 5 : 4);  // log2(16*TM)
  static_assert(TM == 1 || TM == 2 || TM == 4, "TM");
  constexpr int STAGE = (BM + BN) * 8;  // u32x4 slots per stage

  extern __shared__ u32x4_t lds[];

  const int logical = xcd_logical_block(blockIdx.x, per_xcd);
  if (logical >= total) return;
  const int per_plane = tiles_m * tiles_n;
  const int plane = logical / per_plane;
  const int rem = logical - plane * per_plane;
  const int tm = rem / tiles_n, tn = rem - tm * tiles_n;

  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63, l32 = lane & 31, lh = lane >> 5;
  const int wm0 = (wave / WAVES_N) * WM, wn0 = (wave % WAVES_N) * WN;

  const size_t plane_off = (size_t)plane * Np * Np;
  const bf16_t* gm = pm + plane_off;
  const bf16_t* gn = pn + plane_off;

  // ---- global -> register staging: thread covers row (tid/8 + 32*rr), chunk tid%8
  constexpr int RM = BM / 32, RN = BN / 32;
  const int ld_row = tid >> 3, ld_chunk = tid & 7;
  const bf16_t* src_m[RM];
  const bf16_t* src_n[RN];
  int dst_m[RM], dst_n[RN];
#pragma unroll
  for (int r = 0; r < RM; ++r) {
    const int row = ld_row + 32 * r;
    int grow = tm * BM + row;
    grow = grow < Np ? grow : Np - 1;
    src_m[r] = gm + (size_t)grow * Np + ld_chunk * 8;
    dst_m[r] = row * 8 + (ld_chunk ^ key_m<HB>(row));
  }
#pragma unroll
  for (int r = 0; r < RN; ++r) {
    const int row = ld_row + 32 * r;
    int grow = tn * BN + row;
    grow = grow < Np ? grow : Np - 1;
    src_n[r] = gn + (size_t)grow * Np + ld_chunk * 8;
    dst_n[r] = BM * 8 + row * 8 + (ld_chunk ^ key_n(row));
  }

  // ---- MFMA operand fetch addresses (slot of chunk 0; chunk index XOR-ed per k-step)
  int am_row[TM], am_key[TM], bn_row[TN], bn_key[TN];
  {
    const int g = l32 >> 3, hb = (l32 >> 2) & 1, e = l32 & 3;
#pragma unroll
    for (int mt = 0; mt < TM; ++mt) {
      const int row = wm0 + 16 * TM * hb + 16 * mt + 4 * g + e;
      am_row[mt] = row * 8;
      am_key[mt] = key_m<HB>(row);
    }
#pragma unroll
    for (int nt = 0; nt < TN; ++nt) {
      const int row = wn0 + 32 * nt + l32;
      bn_row[nt] = BM * 8 + row * 8;
      bn_key[nt] = key_n(row);
    }
  }

  f32x16_t acc[TM][TN];
#pragma unroll
  for (int mt = 0; mt < TM; ++mt)
#pragma unroll
    for (int nt = 0; nt < TN; ++nt) acc[mt][nt] = zero16();

  u32x4_t st_m[RM], st_n[RN];
  const int nk = Np / kBK;

  // prologue: stage 0
#pragma unroll
  for (int r = 0; r < RM; ++r) st_m[r] = *reinterpret_cast<const u32x4_t*>(src_m[r]);
#pragma unroll
  for (int r = 0; r < RN; ++r) st_n[r] = *reinterpret_cast<const u32x4_t*>(src_n[r]);
#pragma unroll
  for (int r = 0; r < RM; ++r) lds[dst_m[r]] = st_m[r];
#pragma unroll
  for (int r = 0; r < RN; ++r) lds[dst_n[r]] = st_n[r];
  __syncthreads();

  for (int kt = 0; kt < nk; ++kt) {
    const u32x4_t* cur = lds + (kt & 1) * STAGE;
    u32x4_t* nxt = lds + ((kt + 1) & 1) * STAGE;
    const bool more = (kt + 1) < nk;
    if (more) {
      const int koff = (kt + 1) * kBK;
#pragma unroll
      for (int r = 0; r < RM; ++r) st_m[r] = *reinterpret_cast<const u32x4_t*>(src_m[r] + koff);
#pragma unroll
      for (int r = 0; r < RN; ++r) st_n[r] = *reinterpret_cast<const u32x4_t*>(src_n[r] + koff);
    }
#pragma unroll
    for (int ks = 0; ks < kBK / 16; ++ks) {
      const int ch = 2 * ks + lh;
      u32x4_t af[TM], bfr[TN];
#pragma unroll
      for (int mt = 0; mt < TM; ++mt) af[mt] = cur[am_row[mt] + (ch ^ am_key[mt])];
#pragma unroll
      for (int nt = 0; nt < TN; ++nt) bfr[nt] = cur[bn_row[nt] + (ch ^ bn_key[nt])];
#pragma unroll
      for (int mt = 0; mt < TM; ++mt)
#pragma unroll
        for (int nt = 0; nt < TN; ++nt) acc[mt][nt] = mfma_32x32x16(af[mt], bfr[nt], acc[mt][nt]);
    }
    if (more) {
#pragma unroll
      for (int r = 0; r < RM; ++r) nxt[dst_m[r]] = st_m[r];
#pragma unroll
      for (int r = 0; r < RN; ++r) nxt[dst_n[r]] = st_n[r];
    }
    __syncthreads();
  }

  // ---- epilogue: lane (i = column l32, half lh) owns j = j0 + 16*mt + v
  bf16_t* xo = x + plane_off;
#pragma unroll
  for (int nt = 0; nt < TN; ++nt) {
    const int i = tn * BN + wn0 + 32 * nt + l32;
    if (i >= Np) continue;
#pragma unroll
    for (int mt = 0; mt < TM; ++mt) {
      const int j = tm * BM + wm0 + 16 * TM * lh + 16 * mt;
      if (j >= Np) continue;
      u32x4_t lo, hi;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        lo[q] = pack_bf16(acc[mt][nt][2 * q], acc[mt][nt][2 * q + 1]);
        hi[q] = pack_bf16(acc[mt][nt][8 + 2 * q], acc[mt][nt][8 + 2 * q + 1]);
      }
      u32x4_t* dst = reinterpret_cast<u32x4_t*>(xo + (size_t)i * Np + j);
      dst[0] = lo;
      dst[1] = hi;
    }
  }
}

template <int BM, int BN, int WAVES_M, int WAVES_N>
hipError_t launch_contract(const bf16_t* a, const bf16_t* b, bf16_t* x, int planes, int Np, hipStream_t stream) {
  auto kern = contract_kernel<BM, BN, WAVES_M, WAVES_N>;
  const int tiles_m = (Np + BM - 1) / BM, tiles_n = (Np + BN - 1) / BN;
  const long total = (long)planes * tiles_m * tiles_n;
  const int per_xcd = (int)((total + 7) / 8);
  const size_t smem = 2 * (size_t)(BM + BN) * 8 * sizeof(u32x4_t);
  static bool attr_set = false;  // idempotent; a race only repeats the same call
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) return e;
    attr_set = true;
  }
  // M side (register-contiguous output index j) is b, N side (lane index i) is a
  hipLaunchKernelGGL(kern, dim3(per_xcd * 8), dim3(256), smem, stream, b, a, x, Np, tiles_m, tiles_n, (int)total,
                     per_xcd);
  return hipGetLastError();
}

}  // namespace

hipError_t trimul_contract_launch(const bf16_t* a, const bf16_t* b, bf16_t* x, int planes, int Np, int variant,
                                  hipStream_t stream) {
  switch (variant) {
    case 1:
      return launch_contract<128, 128, 2, 2>(a, b, x, planes, Np, stream);
    case 2:
      return launch_contract<256, 128, 2, 2>(a, b, x, planes, Np, stream);
    case 3:
      return launch_contract<256, 256, 2, 2>(a, b, x, planes, Np, stream);
    default:
      return hipErrorInvalidValue;
  }
}

}  // namespace of3

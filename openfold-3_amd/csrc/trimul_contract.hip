// Triangle-multiplication contraction: for every (batch, channel) plane
//     X[i][j] = sum_k A[i][k] * Bm[j][k]
// i.e. the reference's per-channel matrix product of _combine_projections
// (triangular_multiplicative_update.py:71-97).  The projection pass has already laid both
// operands out k-contiguous for either direction, so one "row times row" kernel serves the
// outgoing and the incoming update.
//
// Operand layout ("k-panels"): plane[kb][row][32] bf16 with kb = k / 32, Np rows per panel.
// The 16 rows x 32 k-values that one direct-to-LDS wave instruction moves are then 1 KB of
// contiguous memory, and a whole pipeline stage is two contiguous runs.
// Output layout: plain row-major X[plane][i][j], Np x Np.
//
// Organisation (MFMA-bound kernel, tuned for the MI355X memory system):
//  * persistent work-groups (one per CU, 4 waves, each wave a 128 x BN/2 sub-tile held in
//    AGPRs) walk a list of 256 x BN output tiles; tiles of one plane are dealt to
//    work-groups of one XCD so that operand re-reads hit that XCD's L2;
//  * operands stream global -> LDS with direct-to-LDS loads (no VGPR staging) through a
//    ring of 4 stages of 32 k-values that runs across tile boundaries, so the next tile's
//    operands are in flight while a tile's accumulators are converted and stored;
//  * one barrier per stage, placed between the stage's two k-steps: by then every wave
//    holds the stage's last fragments in registers, so the stage's buffer is refilled at
//    once (stage s+4) and the first fragments of stage s+1 are fetched under the second
//    k-step's MFMAs; the refill's loads are issued one by one between those MFMAs;
//  * the k-blocks of a tile are visited in rotated order, starting at (tm + tn) mod 4:
//    tiles that share operand rows never ask for the same cache line at the same time (the
//    first asks HBM, the others find the line in L2 a stage or two later);
//  * the j side is the MFMA M side with permuted rows so that a lane ends up owning 64
//    consecutive j of one output row; the epilogue transposes 32-row blocks through a
//    wave-private LDS region and stores whole 256-byte row segments.
//
// LDS layout of a stage: rows of 4 chunks of 16 bytes, slot = row*4 + (chunk ^ key(row)).
// A direct-to-LDS instruction fills 64 consecutive slots (lane l -> slot base + l), so the
// lane chooses its *global* chunk as chunk' ^ key(row).
#include "of3_device.h"
#include "of3_kernels.h"
#include "of3_launch.h"

#include <type_traits>

namespace of3 {

namespace {

#define OF3_GLOBAL_AS __attribute__((address_space(1)))
#define OF3_LDS_AS __attribute__((address_space(3)))

constexpr int kBK = 32;  // k per stage = one k-panel

// j side: rows are read in the permuted order {x..x+3, x+64..x+67, x+4..}: (row&1, key)
// must differ within each group of 8 and (row&3, key) within each group of 16 lanes
__device__ __forceinline__ int key_m(int row) { return (((row >> 1) ^ (row >> 2)) & 1) | (((row >> 6) & 1) << 1); }
// i side: natural rows
__device__ __forceinline__ int key_n(int row) { return ((row >> 1) ^ (row >> 3)) & 3; }

__device__ __forceinline__ void compiler_fence() { __asm__ volatile("" ::: "memory"); }

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  // gfx9 encoding: vmcnt[3:0] | expcnt[6:4]=7 | lgkmcnt[11:8]=15 | vmcnt[5:4] at [15:14]
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
  __builtin_amdgcn_s_waitcnt((N & 15) | 0x70 | 0xF00 | ((N >> 4) << 14));
}

template <int BN, int kNS>
__global__ __launch_bounds__(256, 1) void contract_kernel(const bf16_t* __restrict__ pm,  // j side planes (b)
                                                          const bf16_t* __restrict__ pn,  // i side planes (a)
                                                          bf16_t* __restrict__ x, int Np, int nk, int tiles_m,
                                                          int tiles_n, int total_tiles, int tiles_per_xcd) {
  constexpr int BM = 256;
  constexpr int WM = BM / 2, WN = BN / 2;
  constexpr int TM = WM / 32, TN = WN / 32;
  static_assert(TM == 4, "a wave's j range is 128 wide");
  constexpr int ROWS = BM + BN;
  constexpr int STAGE = ROWS * 4;       // u32x4 slots per stage
  constexpr int MI = BM / 16 / 4;       // j-side direct-to-LDS instructions per wave (16 rows each)
  constexpr int NI = BN / 16 / 4;       // i-side
  constexpr int IPW = MI + NI;
  constexpr int NMMA = TM * TN;
  static_assert(IPW <= NMMA, "a stage's loads are issued between the MFMAs of one k-step");
  static_assert((kNS - 2) * IPW + 8 * TN < 64, "vmcnt budget");

  extern __shared__ u32x4_t lds[];

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform, kept in an SGPR
  const int lane = tid & 63, l32 = lane & 31, lh = lane >> 5;
  const int wm0 = (wave >> 1) * WM, wn0 = (wave & 1) * WN;

  // ---- tile list of this work-group: XCD x owns logical tiles [x*tiles_per_xcd, ...)
  const int xcd = blockIdx.x & 7, slot_in_xcd = blockIdx.x >> 3, wgs_per_xcd = gridDim.x >> 3;
  const int xcd_first = xcd * tiles_per_xcd;
  int xcd_count = total_tiles - xcd_first;
  xcd_count = xcd_count < 0 ? 0 : (xcd_count > tiles_per_xcd ? tiles_per_xcd : xcd_count);
  const int my_tiles = slot_in_xcd < xcd_count ? (xcd_count - slot_in_xcd + wgs_per_xcd - 1) / wgs_per_xcd : 0;
  if (my_tiles == 0) return;
  const int per_plane = tiles_m * tiles_n;
  // nk: the 32-wide k-panels that hold keys below N (the panels after them hold zeros and are left out)
  const size_t panel_bytes = (size_t)Np * kBK * 2;

  auto tile_coords = [&](int t_local, int& plane, int& tm, int& tn) {
    const int logical = xcd_first + slot_in_xcd + t_local * wgs_per_xcd;
    plane = logical / per_plane;
    const int rem = logical - plane * per_plane;
    tm = rem / tiles_n;
    tn = rem - tm * tiles_n;
  };

  // ---- direct-to-LDS issue.  One instruction = 16 rows x 64 bytes (1 KB contiguous in a
  // k-panel); lane l -> row l/4, LDS chunk' = l%4, global chunk = chunk' ^ key(row).  The key
  // depends on the lane and on one bit of the (wave-uniform) row block, so two per-lane byte
  // offsets per side serve every instruction; everything else lives in scalar registers.
  const int lrow = lane >> 2, lchunk = lane & 3;
  const uint32_t off_m[2] = {(uint32_t)(lrow * 64 + 16 * (lchunk ^ key_m(lrow))),
                             (uint32_t)(lrow * 64 + 16 * (lchunk ^ key_m(lrow + 64)))};
  const uint32_t off_n[2] = {(uint32_t)(lrow * 64 + 16 * (lchunk ^ key_n(lrow))),
                             (uint32_t)(lrow * 64 + 16 * (lchunk ^ key_n(lrow + 16)))};
  const char* dma_base[IPW];  // first row of each 16-row block in panel 0 of the tile being loaded
  int issue_tile = 0, issue_kb = 0, issue_left = nk, issue_buf = 0;
  auto dma_setup_tile = [&](int t_local) {
    int plane, tm, tn;
    tile_coords(t_local < my_tiles ? t_local : my_tiles - 1, plane, tm, tn);  // past the end: reload the last tile
    const size_t plane_off = (size_t)plane * Np * Np * 2;
    // blocks of padding rows take the last rows with tokens again (of3_tiles.h)
#pragma unroll
    for (int n = 0; n < MI; ++n) {
      const int row = contract_rows_first(tm * BM, 16 * (wave * MI + n), 32 * nk);
      dma_base[n] = reinterpret_cast<const char*>(pm) + plane_off + (size_t)row * (kBK * 2);
    }
#pragma unroll
    for (int n = 0; n < NI; ++n) {
      const int row = contract_rows_first(tn * BN, 16 * (wave * NI + n), 32 * nk);
      dma_base[MI + n] = reinterpret_cast<const char*>(pn) + plane_off + (size_t)row * (kBK * 2);
    }
    issue_kb = ((tm + tn) & 3) % nk;  // rotated start (a small spread keeps the sharers' lines in L2)
    issue_left = nk;
  };
  auto issue_one = [&](int n) {
    u32x4_t* buf = lds + issue_buf * STAGE;
    const char* src = dma_base[n] + (size_t)issue_kb * panel_bytes;
    if (n < MI) {
      const int rb = 16 * (wave * MI + n);
      __builtin_amdgcn_global_load_lds((const void OF3_GLOBAL_AS*)(src + off_m[(rb >> 6) & 1]),
                                       (void OF3_LDS_AS*)(buf + rb * 4), 16, 0, 0);
    } else {
      const int rb = 16 * (wave * NI + (n - MI));
      __builtin_amdgcn_global_load_lds((const void OF3_GLOBAL_AS*)(src + off_n[(rb >> 4) & 1]),
                                       (void OF3_LDS_AS*)(buf + (BM + rb) * 4), 16, 0, 0);
    }
  };
  auto issue_advance = [&]() {
    issue_buf = issue_buf + 1 == kNS ? 0 : issue_buf + 1;
    issue_kb = issue_kb + 1 == nk ? 0 : issue_kb + 1;
    if (--issue_left == 0) dma_setup_tile(++issue_tile);
  };

  // ---- MFMA operand fetch slots.  k-step ks, lane-half lh reads chunk (2*ks + lh) ^ key;
  // row*4 has its two low bits clear, so slot(ks) = slot(0) ^ (2*ks).
  int am_slot[TM], bn_slot[TN];
  {
    const int g = l32 >> 3, hb = (l32 >> 2) & 1, e = l32 & 3;
#pragma unroll
    for (int mt = 0; mt < TM; ++mt) {
      const int row = wm0 + 16 * TM * hb + 16 * mt + 4 * g + e;
      am_slot[mt] = row * 4 + (lh ^ key_m(row));
    }
#pragma unroll
    for (int nt = 0; nt < TN; ++nt) {
      const int row = wn0 + 32 * nt + l32;
      bn_slot[nt] = (BM + row) * 4 + (lh ^ key_n(row));
    }
  }
  auto fetch = [&](const u32x4_t* buf, int ks, u32x4_t (&af)[TM], u32x4_t (&bfr)[TN]) {
#pragma unroll
    for (int mt = 0; mt < TM; ++mt) af[mt] = buf[am_slot[mt] ^ (2 * ks)];
#pragma unroll
    for (int nt = 0; nt < TN; ++nt) bfr[nt] = buf[bn_slot[nt] ^ (2 * ks)];
  };

  f32x16_t acc[TM][TN];
#pragma unroll
  for (int mt = 0; mt < TM; ++mt)
#pragma unroll
    for (int nt = 0; nt < TN; ++nt) acc[mt][nt] = zero16();
  auto mma = [&](const u32x4_t (&af)[TM], const u32x4_t (&bfr)[TN]) {
#pragma unroll
    for (int mt = 0; mt < TM; ++mt)
#pragma unroll
      for (int nt = 0; nt < TN; ++nt) acc[mt][nt] = mfma_32x32x16(af[mt], bfr[nt], acc[mt][nt]);
  };
  // the same, with the refill's loads issued in between
  auto mma_and_issue = [&](const u32x4_t (&af)[TM], const u32x4_t (&bfr)[TN]) {
    int n = 0;
#pragma unroll
    for (int mt = 0; mt < TM; ++mt)
#pragma unroll
      for (int nt = 0; nt < TN; ++nt) {
        acc[mt][nt] = mfma_32x32x16(af[mt], bfr[nt], acc[mt][nt]);
        if (n < IPW) issue_one(n++);
      }
    issue_advance();
  };

  // ---- prologue: fill the ring, make stage 0 visible, fetch its first fragments
  dma_setup_tile(0);
#pragma unroll
  for (int s = 0; s < kNS; ++s) {
#pragma unroll
    for (int n = 0; n < IPW; ++n) issue_one(n);
    issue_advance();
  }
  wait_vmcnt<(kNS - 1) * IPW>();
  compiler_fence();
  __builtin_amdgcn_s_barrier();
  compiler_fence();

  u32x4_t a0[TM], b0[TN], a1[TM], b1[TN];
  fetch(lds, 0, a0, b0);

  int cur_buf = 0;
  bool stores_pending = false;  // the previous tile's full set of output stores may still be in the queue
  for (int t_local = 0; t_local < my_tiles; ++t_local) {
    for (int kb = 0; kb < nk; ++kb) {
      const u32x4_t* cur = lds + cur_buf * STAGE;
      // The second k-step's fragments are requested right after the first MFMA: that MFMA
      // carries the wait for a0/b0 (with direct-to-LDS loads in flight every LDS wait the
      // compiler emits is a wait for all outstanding reads), so the new reads travel under the
      // remaining MFMAs instead of being waited for at once.
      acc[0][0] = mfma_32x32x16(a0[0], b0[0], acc[0][0]);
      __builtin_amdgcn_sched_barrier(0);
      fetch(cur, 1, a1, b1);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int mt = 0; mt < TM; ++mt)
#pragma unroll
        for (int nt = 0; nt < TN; ++nt)
          if (mt + nt > 0) acc[mt][nt] = mfma_32x32x16(a0[mt], b0[nt], acc[mt][nt]);
      __builtin_amdgcn_sched_barrier(0);

      // This wave holds all of stage s in registers.  Stages s+1..s+3 are in flight and
      // stage s+1 must have landed, in every wave (hence the barrier).  VMEM operations
      // retire in order, so "at most n outstanding" means everything older than the newest
      // n has completed.  The output stores of a tile that has just ended sit in the same
      // queue behind the loads of three stages; during the next three stages they are
      // simply allowed to stay outstanding, otherwise the wait would drain the whole ring
      // at every tile boundary.
      __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): a1/b1 have arrived
      if (stores_pending && kb < kNS - 1 && nk >= kNS) wait_vmcnt<(kNS - 2) * IPW + 8 * TN>();
      else wait_vmcnt<(kNS - 2) * IPW>();
      compiler_fence();
      __builtin_amdgcn_s_barrier();
      compiler_fence();
      __builtin_amdgcn_sched_barrier(0);

      // after the barrier no wave reads the buffer of stage s any more: refill it with
      // stage s+4 while the second k-step's MFMAs run
      cur_buf = cur_buf + 1 == kNS ? 0 : cur_buf + 1;
      fetch(lds + cur_buf * STAGE, 0, a0, b0);  // after the last stage this reads data that is never used
      mma_and_issue(a1, b1);
      __builtin_amdgcn_sched_barrier(0);
    }

    // ---- tile finished.  Each wave transposes its 32-row blocks through a private 8 KB
    // LDS region (row-major [32 i][128 j] bf16, 16-byte chunks XOR-swizzled by the row) and
    // writes whole 256-byte row segments.
    int plane, tm, tn;
    tile_coords(t_local, plane, tm, tn);
    bf16_t* xo = x + (size_t)plane * Np * Np;
    u32x4_t* epi = lds + kNS * STAGE + wave * 512;
    const int jbase = tm * BM + wm0;
    int n_stores = 0;
#pragma unroll
    for (int nt = 0; nt < TN; ++nt) {
#pragma unroll
      for (int mt = 0; mt < TM; ++mt) {
        u32x4_t lo, hi;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          lo[q] = pack_bf16(acc[mt][nt][2 * q], acc[mt][nt][2 * q + 1]);
          hi[q] = pack_bf16(acc[mt][nt][8 + 2 * q], acc[mt][nt][8 + 2 * q + 1]);
        }
        const int chunk = 8 * lh + 2 * mt;  // j-local = 64*lh + 16*mt + (0..15)
        epi[l32 * 16 + (chunk ^ (l32 & 7))] = lo;
        epi[l32 * 16 + ((chunk + 1) ^ (l32 & 7))] = hi;
        acc[mt][nt] = zero16();
      }
      // Only the rows and columns below Nr = 32 * nk (the tokens, rounded up to whole 32-blocks) are ever
      // read: a 32-row block is entirely below it or entirely above (wave-uniform), the wave's 128 columns
      // may straddle it (then the lanes decide, and the stores are not counted)
      const int i0 = tn * BN + wn0 + 32 * nt;
      const int Nr = 32 * nk;
      if (i0 < Nr && jbase + WM <= Nr) {
#pragma unroll
        for (int rr = 0; rr < 8; ++rr) {
          const int row = 4 * rr + (lane >> 4), chunk = lane & 15;
          const u32x4_t v = epi[row * 16 + (chunk ^ (row & 7))];
          *reinterpret_cast<u32x4_t*>(xo + (size_t)(i0 + row) * Np + jbase + 8 * chunk) = v;
        }
        n_stores += 8;
      } else if (i0 < Nr && jbase < Nr) {
#pragma unroll
        for (int rr = 0; rr < 8; ++rr) {
          const int row = 4 * rr + (lane >> 4), chunk = lane & 15;
          const u32x4_t v = epi[row * 16 + (chunk ^ (row & 7))];
          if (jbase + 8 * chunk < Nr) *reinterpret_cast<u32x4_t*>(xo + (size_t)(i0 + row) * Np + jbase + 8 * chunk) = v;
        }
      }
      __builtin_amdgcn_sched_barrier(0);  // one block at a time keeps the live registers low
    }
    // only a complete set of stores is accounted for exactly; otherwise the next waits
    // simply cover them too (waiting for more than necessary is always safe)
    stores_pending = (n_stores == 8 * TN);
  }
  wait_vmcnt<0>();  // loads issued past the end must not outlive the work-group's LDS
}

template <int BN, int kNS>
hipError_t launch_contract(const bf16_t* a, const bf16_t* b, bf16_t* x, int planes, int Np, int nk, hipStream_t stream) {
  constexpr int BM = 256;
  auto kern = contract_kernel<BN, kNS>;
  const size_t smem = ((size_t)kNS * (BM + BN) * 4 + 4 * 512) * sizeof(u32x4_t);  // ring + epilogue staging
  static int cache[kMaxDevices];
  int cus = 0;
  hipError_t e = per_device(
      cache,
      [&](int dev, int* v) {
        hipError_t s = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
        return s != hipSuccess ? s : cu_count(dev, v);
      },
      &cus);
  if (e != hipSuccess) return e;
  const int tiles_m = (Np + BM - 1) / BM, tiles_n = (Np + BN - 1) / BN;
  const int total = planes * tiles_m * tiles_n;
  const int tiles_per_xcd = (total + 7) / 8;
  int grid = (cus / 8) * 8;  // a multiple of the 8 XCDs
  if (grid < 8) grid = 8;
  // M side (register-contiguous output index j) is b, N side (lane index i) is a
  hipLaunchKernelGGL(kern, dim3(grid), dim3(256), smem, stream, b, a, x, Np, nk, tiles_m, tiles_n, total, tiles_per_xcd);
  return hipGetLastError();
}


// ---- eight-wave organisation: 384 x 192 output tiles ------------------------------------------
// A plane of 768 x 768 is 2 x 4 = 8 such tiles, so the 32 work-groups of an XCD finish whole planes
// together (4 per round) and no operand panel is fetched from HBM by two rounds; a tile moves 14 %
// fewer operand bytes from L2 per flop than a 256 x 192 one.  Eight waves (4 along j x 2 along i),
// each a 96 x 96 sub-tile (144 accumulator registers), two per SIMD; the ring has three stages of
// 36 KB.  Both sides keep their natural row order; a lane therefore holds runs of 4 consecutive j,
// which the epilogue writes as 8-byte pieces into a wave-private [32 i][96 j] staging block (chunk
// index XOR (i / 4) % 4 within each group of four: conflict-free for the writers) and reads back as
// whole 192-byte row segments.
// A stage is 24 + 12 direct-to-LDS instructions: three j-side ones per wave, two i-side ones for
// waves 0..3 and one for waves 4..7 (a wave-uniform difference, so every wait stays a constant).
template <int kNS>
__global__ __launch_bounds__(512, 1) void contract8_kernel(const bf16_t* __restrict__ pm,  // j side planes (b)
                                                           const bf16_t* __restrict__ pn,  // i side planes (a)
                                                           bf16_t* __restrict__ x, int Np, int nk, int tiles_m,
                                                           int tiles_n, int total_tiles, int tiles_per_xcd) {
  constexpr int BM = 384, BN = 192;
  constexpr int WM = 96, WN = 96;
  constexpr int TM = WM / 32, TN = WN / 32;
  constexpr int ROWS = BM + BN;
  constexpr int STAGE = ROWS * 4;
  constexpr int MI = BM / 16 / 8;           // 3 j-side instructions per wave
  constexpr int NI_LO = 2, NI_HI = 1;       // i-side instructions of waves 0..3 / 4..7
  constexpr int IPW_LO = MI + NI_LO, IPW_HI = MI + NI_HI;
  constexpr int NMMA = TM * TN;
  constexpr int EPI_ROW = 12;               // 16-byte slots per staging row
  constexpr int EPI_WAVE = 32 * EPI_ROW;    // slots per wave
  constexpr int STORES = 6 * TN;            // output stores of a wave per tile
  static_assert(IPW_LO <= NMMA, "a stage's loads are issued between the MFMAs of one k-step");
  static_assert((kNS - 2) * IPW_LO + STORES < 64, "vmcnt budget");

  extern __shared__ u32x4_t lds[];

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const bool lo_wave = wave < 4;
  const int lane = tid & 63, l32 = lane & 31, lh = lane >> 5;
  const int wm0 = (wave >> 1) * WM, wn0 = (wave & 1) * WN;

  const int xcd = blockIdx.x & 7, slot_in_xcd = blockIdx.x >> 3, wgs_per_xcd = gridDim.x >> 3;
  const int xcd_first = xcd * tiles_per_xcd;
  int xcd_count = total_tiles - xcd_first;
  xcd_count = xcd_count < 0 ? 0 : (xcd_count > tiles_per_xcd ? tiles_per_xcd : xcd_count);
  const int my_tiles = slot_in_xcd < xcd_count ? (xcd_count - slot_in_xcd + wgs_per_xcd - 1) / wgs_per_xcd : 0;
  if (my_tiles == 0) return;
  const int per_plane = tiles_m * tiles_n;
  // nk: the 32-wide k-panels that hold keys below N (the panels after them hold zeros and are left out)
  const size_t panel_bytes = (size_t)Np * kBK * 2;

  auto tile_coords = [&](int t_local, int& plane, int& tm, int& tn) {
    const int logical = xcd_first + slot_in_xcd + t_local * wgs_per_xcd;
    plane = logical / per_plane;
    const int rem = logical - plane * per_plane;
    tm = rem / tiles_n;
    tn = rem - tm * tiles_n;
  };

  // row block (16 rows) that instruction n of this wave fills, counted within its side
  auto block_row = [&](int n) {
    if (n < MI) return 16 * (wave * MI + n);
    return lo_wave ? 16 * (wave * NI_LO + (n - MI)) : 16 * (4 * NI_LO + (wave - 4));
  };
  const int lrow = lane >> 2, lchunk = lane & 3;
  const uint32_t off[2] = {(uint32_t)(lrow * 64 + 16 * (lchunk ^ key_n(lrow))),
                           (uint32_t)(lrow * 64 + 16 * (lchunk ^ key_n(lrow + 16)))};
  const char* dma_base[IPW_LO];
  int issue_tile = 0, issue_kb = 0, issue_left = nk, issue_buf = 0;
  auto dma_setup_tile = [&](int t_local) {
    int plane, tm, tn;
    tile_coords(t_local < my_tiles ? t_local : my_tiles - 1, plane, tm, tn);  // past the end: reload the last tile
    const size_t plane_off = (size_t)plane * Np * Np * 2;
    // blocks of padding rows take the last rows with tokens again (of3_tiles.h)
#pragma unroll
    for (int n = 0; n < IPW_LO; ++n) {
      const bf16_t* side = n < MI ? pm : pn;
      const int row = contract_rows_first(n < MI ? tm * BM : tn * BN, block_row(n), 32 * nk);
      dma_base[n] = reinterpret_cast<const char*>(side) + plane_off + (size_t)row * (kBK * 2);
    }
    issue_kb = ((tm + tn) & 3) % nk;
    issue_left = nk;
  };
  auto issue_one = [&](int n) {  // n is a constant at every call site; the fifth one belongs to waves 0..3 only
    if (n == IPW_LO - 1 && !lo_wave) return;
    u32x4_t* buf = lds + issue_buf * STAGE;
    const char* src = dma_base[n] + (size_t)issue_kb * panel_bytes;
    const int rb = block_row(n);
    __builtin_amdgcn_global_load_lds((const void OF3_GLOBAL_AS*)(src + off[(rb >> 4) & 1]),
                                     (void OF3_LDS_AS*)(buf + ((n < MI ? 0 : BM) + rb) * 4), 16, 0, 0);
  };
  auto issue_advance = [&]() {
    issue_buf = issue_buf + 1 == kNS ? 0 : issue_buf + 1;
    issue_kb = issue_kb + 1 == nk ? 0 : issue_kb + 1;
    if (--issue_left == 0) dma_setup_tile(++issue_tile);
  };
  // "at most `stages` whole stages of this wave's loads (plus `extra` stores) still outstanding"
  auto wait_stages = [&](auto stages, auto extra) {
    constexpr int S = decltype(stages)::value, E = decltype(extra)::value;
    if (lo_wave) wait_vmcnt<S * IPW_LO + E>();
    else wait_vmcnt<S * IPW_HI + E>();
  };

  int am_slot[TM], bn_slot[TN];
#pragma unroll
  for (int mt = 0; mt < TM; ++mt) {
    const int row = wm0 + 32 * mt + l32;
    am_slot[mt] = row * 4 + (lh ^ key_n(row));
  }
#pragma unroll
  for (int nt = 0; nt < TN; ++nt) {
    const int row = wn0 + 32 * nt + l32;
    bn_slot[nt] = (BM + row) * 4 + (lh ^ key_n(row));
  }
  auto fetch = [&](const u32x4_t* buf, int ks, u32x4_t (&af)[TM], u32x4_t (&bfr)[TN]) {
#pragma unroll
    for (int mt = 0; mt < TM; ++mt) af[mt] = buf[am_slot[mt] ^ (2 * ks)];
#pragma unroll
    for (int nt = 0; nt < TN; ++nt) bfr[nt] = buf[bn_slot[nt] ^ (2 * ks)];
  };

  f32x16_t acc[TM][TN];
#pragma unroll
  for (int mt = 0; mt < TM; ++mt)
#pragma unroll
    for (int nt = 0; nt < TN; ++nt) acc[mt][nt] = zero16();
  auto mma_and_issue = [&](const u32x4_t (&af)[TM], const u32x4_t (&bfr)[TN]) {
    int n = 0;
#pragma unroll
    for (int mt = 0; mt < TM; ++mt)
#pragma unroll
      for (int nt = 0; nt < TN; ++nt) {
        acc[mt][nt] = mfma_32x32x16(af[mt], bfr[nt], acc[mt][nt]);
        if (n < IPW_LO) issue_one(n++);
      }
    issue_advance();
  };

  dma_setup_tile(0);
#pragma unroll
  for (int s = 0; s < kNS; ++s) {
#pragma unroll
    for (int n = 0; n < IPW_LO; ++n) issue_one(n);
    issue_advance();
  }
  wait_stages(std::integral_constant<int, kNS - 1>{}, std::integral_constant<int, 0>{});
  compiler_fence();
  __builtin_amdgcn_s_barrier();
  compiler_fence();

  u32x4_t a0[TM], b0[TN], a1[TM], b1[TN];
  fetch(lds, 0, a0, b0);

  int cur_buf = 0;
  bool stores_pending = false;
  for (int t_local = 0; t_local < my_tiles; ++t_local) {
    for (int kb = 0; kb < nk; ++kb) {
      const u32x4_t* cur = lds + cur_buf * STAGE;
      acc[0][0] = mfma_32x32x16(a0[0], b0[0], acc[0][0]);
      __builtin_amdgcn_sched_barrier(0);
      fetch(cur, 1, a1, b1);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int mt = 0; mt < TM; ++mt)
#pragma unroll
        for (int nt = 0; nt < TN; ++nt)
          if (mt + nt > 0) acc[mt][nt] = mfma_32x32x16(a0[mt], b0[nt], acc[mt][nt]);
      __builtin_amdgcn_sched_barrier(0);

      // as in the four-wave kernel: stage s is in registers, stage s+1 must have landed in every
      // wave, the newest kNS-2 stages (and a finished tile's stores, for its first stages) may
      // stay in flight
      __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): a1/b1 have arrived
      if (stores_pending && kb < kNS - 1 && nk >= kNS)
        wait_stages(std::integral_constant<int, kNS - 2>{}, std::integral_constant<int, STORES>{});
      else
        wait_stages(std::integral_constant<int, kNS - 2>{}, std::integral_constant<int, 0>{});
      compiler_fence();
      __builtin_amdgcn_s_barrier();
      compiler_fence();
      __builtin_amdgcn_sched_barrier(0);

      cur_buf = cur_buf + 1 == kNS ? 0 : cur_buf + 1;
      fetch(lds + cur_buf * STAGE, 0, a0, b0);
      mma_and_issue(a1, b1);
      __builtin_amdgcn_sched_barrier(0);
    }

    // ---- tile finished: 32-row blocks through the wave's staging area, 192-byte row segments out
    int plane, tm, tn;
    tile_coords(t_local, plane, tm, tn);
    bf16_t* xo = x + (size_t)plane * Np * Np;
    u32x2_t* epi2 = reinterpret_cast<u32x2_t*>(lds + kNS * STAGE + wave * EPI_WAVE);
    const u32x4_t* epi4 = lds + kNS * STAGE + wave * EPI_WAVE;
    const int jbase = tm * BM + wm0;
    int n_stores = 0;
#pragma unroll
    for (int nt = 0; nt < TN; ++nt) {
#pragma unroll
      for (int mt = 0; mt < TM; ++mt) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {  // registers 4g..4g+3: j-local = 32*mt + 8*g + 4*lh + (0..3) of row i = l32
          const u32x2_t v = {pack_bf16(acc[mt][nt][4 * g], acc[mt][nt][4 * g + 1]),
                             pack_bf16(acc[mt][nt][4 * g + 2], acc[mt][nt][4 * g + 3])};
          epi2[(l32 * EPI_ROW + 4 * mt + (g ^ ((l32 >> 2) & 3))) * 2 + lh] = v;
        }
        acc[mt][nt] = zero16();
      }
      const int i0 = tn * BN + wn0 + 32 * nt;
      const int Nr = 32 * nk;  // the tokens, rounded up to whole 32-blocks: nothing beyond is ever read
      const bool whole = i0 + 32 <= Nr && jbase + WM <= Nr;  // wave-uniform
#pragma unroll
      for (int rr = 0; rr < 6; ++rr) {
        const int idx = 64 * rr + lane, row = idx / 12, chunk = idx - 12 * row;
        const u32x4_t v = epi4[row * EPI_ROW + (chunk ^ ((row >> 2) & 3))];
        if (whole || (i0 + row < Nr && jbase + 8 * chunk < Nr))
          *reinterpret_cast<u32x4_t*>(xo + (size_t)(i0 + row) * Np + jbase + 8 * chunk) = v;
      }
      if (whole) n_stores += 6;
      __builtin_amdgcn_sched_barrier(0);
    }
    // only a complete set of unconditional stores is accounted for exactly; otherwise the next
    // waits simply cover them too
    stores_pending = (n_stores == STORES);
  }
  wait_vmcnt<0>();
}

template <int kNS>
hipError_t launch_contract8(const bf16_t* a, const bf16_t* b, bf16_t* x, int planes, int Np, int nk, hipStream_t stream) {
  constexpr int BM = 384, BN = 192;
  auto kern = contract8_kernel<kNS>;
  const size_t smem = ((size_t)kNS * (BM + BN) * 4 + 8 * 32 * 12) * sizeof(u32x4_t);  // ring + epilogue staging
  static int cache[kMaxDevices];
  int cus = 0;
  hipError_t e = per_device(
      cache,
      [&](int dev, int* v) {
        hipError_t s = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
        return s != hipSuccess ? s : cu_count(dev, v);
      },
      &cus);
  if (e != hipSuccess) return e;
  const int tiles_m = (Np + BM - 1) / BM, tiles_n = (Np + BN - 1) / BN;
  const int total = planes * tiles_m * tiles_n;
  const int tiles_per_xcd = (total + 7) / 8;
  int grid = (cus / 8) * 8;
  if (grid < 8) grid = 8;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(512), smem, stream, b, a, x, Np, nk, tiles_m, tiles_n, total, tiles_per_xcd);
  return hipGetLastError();
}

}  // namespace

hipError_t trimul_contract_launch(const bf16_t* a, const bf16_t* b, bf16_t* x, int planes, int Np, int nk, int variant,
                                  hipStream_t stream) {
  if (nk < 1 || nk > Np / kBK) return hipErrorInvalidValue;
  switch (variant) {
    case 1:
      return launch_contract<192, 4>(a, b, x, planes, Np, nk, stream);
    case 2:
      return launch_contract<128, 4>(a, b, x, planes, Np, nk, stream);
    case 3:
      return launch_contract<256, 4>(a, b, x, planes, Np, nk, stream);
    case 4:
      return launch_contract8<3>(a, b, x, planes, Np, nk, stream);
    default:
      return hipErrorInvalidValue;
  }
}

}  // namespace of3

// Triangle-multiplication contraction, large-N variant: same arithmetic as
// trimul_contract.hip (X[i][j] = sum_k A[i][k] * Bm[j][k] per (batch, channel) plane,
// triangular_multiplicative_update.py:71-97), organised for the MI355X memory system:
//
//  * persistent work-groups (one per CU, 4 waves, each wave a 128 x (BN/2) sub-tile held in
//    AGPRs) walk a list of BM x BN output tiles; tiles of one plane are dealt to
//    work-groups of one XCD so that the operand re-reads hit that XCD's L2;
//  * operands stream global -> LDS with direct-to-LDS loads (global_load_lds_dwordx4, no
//    VGPR staging) through a ring of NS stages of 32 k-values; the ring runs across tile
//    boundaries, so the next tile's operands are already in flight while a tile's
//    accumulators are converted and stored;
//  * one barrier per stage, placed in the middle of the stage's MFMA work: by then every
//    wave holds the stage's last fragments in registers, so the stage's LDS buffer can be
//    refilled immediately and the first fragments of the next stage are fetched under the
//    remaining MFMAs.
//
// LDS layout of a stage: rows of 32 k-values = 4 chunks of 16 bytes, slot = row*4 +
// (chunk ^ key(row)).  A direct-to-LDS wave instruction fills 64 consecutive slots (lane l
// -> slot base + l), so the lane chooses its *global* chunk as chunk' ^ key(row).
#include "of3_device.h"
#include "of3_kernels.h"

namespace of3 {

namespace {

#define OF3_GLOBAL_AS __attribute__((address_space(1)))
#define OF3_LDS_AS __attribute__((address_space(3)))

constexpr int kPBK = 32;  // k per stage
constexpr int kNS = 4;    // ring depth

// j side (MFMA M side, rows permuted so a lane owns 16*TM consecutive j)
template <int HB>
__device__ __forceinline__ int pkey_m(int row) {
  return (((row >> 1) ^ (row >> 2)) & 1) | (((row >> HB) & 1) << 1);
}
// i side: natural rows
__device__ __forceinline__ int pkey_n(int row) { return ((row >> 1) ^ (row >> 3)) & 3; }

__device__ __forceinline__ void compiler_fence() { __asm__ volatile("" ::: "memory"); }

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  // gfx9 encoding: vmcnt[3:0] | expcnt[6:4]=7 | lgkmcnt[11:8]=15 | vmcnt[5:4] at [15:14]
  __builtin_amdgcn_s_waitcnt((N & 15) | 0x70 | 0xF00 | ((N >> 4) << 14));
}

template <int BM, int BN>
__global__ __launch_bounds__(256, 1) void contract_pipe_kernel(const bf16_t* __restrict__ pm,  // j side planes
                                                               const bf16_t* __restrict__ pn,  // i side planes
                                                               bf16_t* __restrict__ x, int Np, int tiles_m,
                                                               int tiles_n, int total_tiles, int tiles_per_xcd) {
  constexpr int WM = BM / 2, WN = BN / 2;
  constexpr int TM = WM / 32, TN = WN / 32;
  static_assert(TM == 4, "j side of a wave is 128 wide");
  constexpr int HB = 6;                         // log2(16*TM)
  constexpr int ROWS = BM + BN;                 // LDS rows per stage
  constexpr int STAGE = ROWS * 4;               // u32x4 slots per stage
  constexpr int INSTR = ROWS / 16;              // direct-to-LDS wave instructions per stage
  constexpr int IPW = INSTR / 4;                // per wave
  static_assert(INSTR % 4 == 0, "stage must split evenly over 4 waves");

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
  const int nk = Np / kPBK;
  const int total_stages = my_tiles * nk;

  auto tile_coords = [&](int t_local, int& plane, int& tm, int& tn) {
    const int logical = xcd_first + slot_in_xcd + t_local * wgs_per_xcd;
    plane = logical / per_plane;
    const int rem = logical - plane * per_plane;
    tm = rem / tiles_n;
    tn = rem - tm * tiles_n;
  };

  // ---- direct-to-LDS issue state.  Wave w, instruction n fills stage rows
  // 16*(w*IPW+n) .. +15; lane -> (row, chunk'), global chunk = chunk' ^ key(row).
  const bf16_t* dma_src[IPW];
  int issue_tile = 0, issue_kb = 0, issue_buf = 0;
  auto dma_setup_tile = [&](int t_local) {
    int plane, tm, tn;
    tile_coords(t_local, plane, tm, tn);
    const size_t plane_off = (size_t)plane * Np * Np;
#pragma unroll
    for (int n = 0; n < IPW; ++n) {
      const int row = 16 * (wave * IPW + n) + (lane >> 2);  // [0,BM) j side, [BM,ROWS) i side
      const int cprime = lane & 3;
      const bool is_m = row < BM;
      const int trow = is_m ? row : row - BM;
      const int chunk = cprime ^ (is_m ? pkey_m<HB>(trow) : pkey_n(trow));
      int grow = is_m ? tm * BM + trow : tn * BN + trow;
      grow = grow < Np ? grow : Np - 1;
      dma_src[n] = (is_m ? pm : pn) + plane_off + (size_t)grow * Np + chunk * 8;
    }
  };
  auto issue_stage = [&]() {
    u32x4_t* buf = lds + issue_buf * STAGE + 64 * (wave * IPW);
#pragma unroll
    for (int n = 0; n < IPW; ++n) {
      __builtin_amdgcn_global_load_lds((const void OF3_GLOBAL_AS*)dma_src[n], (void OF3_LDS_AS*)(buf + 64 * n), 16, 0,
                                       0);
      dma_src[n] += kPBK;
    }
    issue_buf = (issue_buf + 1) & (kNS - 1);
    if (++issue_kb == nk) {
      issue_kb = 0;
      ++issue_tile;
      if (issue_tile < my_tiles) dma_setup_tile(issue_tile);
    }
  };

  // ---- MFMA operand fetch slots.  k-step ks, lane-half lh reads chunk (2*ks + lh) ^ key;
  // row*4 has its two low bits clear, so slot(ks) = slot(0) ^ (2*ks).
  int am_slot[TM], bn_slot[TN];
  {
    const int g = l32 >> 3, hb = (l32 >> 2) & 1, e = l32 & 3;
#pragma unroll
    for (int mt = 0; mt < TM; ++mt) {
      const int row = wm0 + 16 * TM * hb + 16 * mt + 4 * g + e;
      am_slot[mt] = row * 4 + (lh ^ pkey_m<HB>(row));
    }
#pragma unroll
    for (int nt = 0; nt < TN; ++nt) {
      const int row = wn0 + 32 * nt + l32;
      bn_slot[nt] = (BM + row) * 4 + (lh ^ pkey_n(row));
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

  // ---- prologue: fill the ring (NS stages), make stage 0 visible, fetch its first fragments
  dma_setup_tile(0);
  int issued = 0;
#pragma unroll
  for (int s = 0; s < kNS; ++s)
    if (s < total_stages) {
      issue_stage();
      ++issued;
    }
  {
    const int later = issued - 1;  // stages that may stay in flight
    if (later >= 3) wait_vmcnt<3 * IPW>();
    else if (later == 2) wait_vmcnt<2 * IPW>();
    else if (later == 1) wait_vmcnt<IPW>();
    else wait_vmcnt<0>();
  }
  compiler_fence();
  __builtin_amdgcn_s_barrier();
  compiler_fence();

  u32x4_t a0[TM], b0[TN], a1[TM], b1[TN];
  fetch(lds, 0, a0, b0);

  int kb = 0, t_local = 0, cur_buf = 0;
  int stores_in_queue = 0, stores_age = 0;  // store instructions of the last epilogue still counted by vmcnt
  for (int s = 0; s < total_stages; ++s) {
    const u32x4_t* cur = lds + cur_buf * STAGE;
    cur_buf = (cur_buf + 1) & (kNS - 1);
    // second half of this stage's fragments, fetched under the first half's MFMAs
    fetch(cur, 1, a1, b1);
#pragma unroll
    for (int mt = 0; mt < TM; ++mt)
#pragma unroll
      for (int nt = 0; nt < TN; ++nt) acc[mt][nt] = mfma_32x32x16(a0[mt], b0[nt], acc[mt][nt]);
    __builtin_amdgcn_sched_barrier(0);

    // This wave now holds all of stage s in registers.  Stages s+1 .. s+NS-1 are in
    // flight; stage s+1 must have landed (in every wave: hence the barrier) before it is
    // read.  VMEM operations retire in order, so "at most n outstanding" means everything
    // older than the newest n has completed.
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): a1/b1 have arrived
    {
      const int remaining = total_stages - (s + 1);  // stages after s
      const int later = (remaining < kNS - 1 ? remaining : kNS - 1) - 1;
      if (remaining > 0) {
        if (later >= 2) {
          // The output stores of a finished tile sit in the same in-order queue, behind
          // the loads of the three stages that were in flight when they were issued.  For
          // the next three stages they are simply allowed to stay outstanding; without
          // that the wait would drain the whole ring at every tile boundary.
          switch (stores_in_queue) {
            case 0: wait_vmcnt<2 * IPW>(); break;
            case 8: wait_vmcnt<2 * IPW + 8>(); break;
            case 16: wait_vmcnt<2 * IPW + 16>(); break;
            case 24: wait_vmcnt<2 * IPW + 24>(); break;
            default: wait_vmcnt<2 * IPW + 32>(); break;
          }
        } else if (later == 1) {
          wait_vmcnt<IPW>();
        } else {
          wait_vmcnt<0>();
        }
      }
      if (stores_age > 0 && --stores_age == 0) stores_in_queue = 0;
    }
    compiler_fence();
    __builtin_amdgcn_s_barrier();
    compiler_fence();
    __builtin_amdgcn_sched_barrier(0);

    // after the barrier no wave reads the buffer of stage s any more: refill it with
    // stage s+NS while the second half of the MFMAs runs
    const bool last_k = (kb == nk - 1);
    if (s + 1 < total_stages) fetch(lds + cur_buf * STAGE, 0, a0, b0);
    if (s + kNS < total_stages) issue_stage();
#pragma unroll
    for (int mt = 0; mt < TM; ++mt)
#pragma unroll
      for (int nt = 0; nt < TN; ++nt) acc[mt][nt] = mfma_32x32x16(a1[mt], b1[nt], acc[mt][nt]);
    __builtin_amdgcn_sched_barrier(0);

    if (last_k) {
      // ---- tile finished.  A lane holds, per 32-row block nt, 64 consecutive j of row
      // i = l32 in 8 pieces of 16 bytes; storing those directly makes every wave store
      // touch 64 different cache lines with 16 bytes each.  Instead each wave transposes
      // the block through a private 8 KB LDS region (row-major [32 i][128 j] bf16, 16-byte
      // chunks XOR-swizzled by the row) and writes whole 256-byte row segments.
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
        // Np is a multiple of 128, so a 32-row block and the wave's 128 columns are
        // either entirely inside the plane or entirely outside: the guard is wave-uniform
        const int i0 = tn * BN + wn0 + 32 * nt;
        if (i0 < Np && jbase < Np) {
#pragma unroll
          for (int rr = 0; rr < 8; ++rr) {
            const int row = 4 * rr + (lane >> 4), chunk = lane & 15;
            const u32x4_t v = epi[row * 16 + (chunk ^ (row & 7))];
            *reinterpret_cast<u32x4_t*>(xo + (size_t)(i0 + row) * Np + jbase + 8 * chunk) = v;
          }
          n_stores += 8;
        }
        __builtin_amdgcn_sched_barrier(0);  // one 32-row block at a time: keeps the live registers low
      }
      stores_in_queue = n_stores;
      stores_age = 3;
      kb = 0;
      ++t_local;
    } else {
      ++kb;
    }
  }
}

// ---------------------------------------------------------------------------------------
// Same organisation with 64 k-values per stage (full 128-byte lines per row: a direct-to-LDS
// load of half a line costs the L1 as much as a whole one) and a two-stage ring.
//
// Per stage: four k-steps of TM*TN MFMAs with double-buffered fragments; the single barrier
// sits before the last k-step's MFMAs, where the wave already holds the stage's last
// fragments, so the stage's buffer can be refilled (stage s+2) and the first fragments of
// stage s+1 fetched under those MFMAs.  The loads of a stage are issued one at a time
// between MFMAs so that their address arithmetic hides in the MFMA issue gaps.
//
// The k-blocks of a tile are visited in rotated order, starting at (tm + tn) mod nk: tiles
// that share operand rows (same tm or same tn) therefore never ask for the same cache line
// at the same time -- the first asks HBM, the others find the line in the XCD's L2 one to
// three stages later -- instead of queueing up behind one outstanding miss.
constexpr int kQBK = 64;

template <int HB>
__device__ __forceinline__ int qkey_m(int row) { return (row & 3) | (((row >> HB) & 1) << 2); }
__device__ __forceinline__ int qkey_n(int row) { return row & 7; }

template <int BM, int BN>
__global__ __launch_bounds__(256, 1) void contract_pipe64_kernel(const bf16_t* __restrict__ pm,
                                                                 const bf16_t* __restrict__ pn,
                                                                 bf16_t* __restrict__ x, int Np, int tiles_m,
                                                                 int tiles_n, int total_tiles, int tiles_per_xcd) {
  constexpr int WM = BM / 2, WN = BN / 2;
  constexpr int TM = WM / 32, TN = WN / 32;
  static_assert(TM == 4, "j side of a wave is 128 wide");
  constexpr int HB = 6;
  constexpr int ROWS = BM + BN;
  constexpr int STAGE = ROWS * 8;       // u32x4 slots per stage
  constexpr int MI = BM / 8 / 4;        // j-side direct-to-LDS instructions per wave (8 rows each)
  constexpr int NI = BN / 8 / 4;        // i-side
  constexpr int IPW = MI + NI;
  constexpr int NMMA = TM * TN;
  static_assert(IPW <= 2 * NMMA, "loads are issued between the MFMAs of one k-step");

  extern __shared__ u32x4_t lds[];

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63, l32 = lane & 31, lh = lane >> 5;
  const int wm0 = (wave >> 1) * WM, wn0 = (wave & 1) * WN;

  const int xcd = blockIdx.x & 7, slot_in_xcd = blockIdx.x >> 3, wgs_per_xcd = gridDim.x >> 3;
  const int xcd_first = xcd * tiles_per_xcd;
  int xcd_count = total_tiles - xcd_first;
  xcd_count = xcd_count < 0 ? 0 : (xcd_count > tiles_per_xcd ? tiles_per_xcd : xcd_count);
  const int my_tiles = slot_in_xcd < xcd_count ? (xcd_count - slot_in_xcd + wgs_per_xcd - 1) / wgs_per_xcd : 0;
  if (my_tiles == 0) return;
  const int per_plane = tiles_m * tiles_n;
  const int nk = Np / kQBK;
  const size_t row_bytes = (size_t)Np * 2;

  auto tile_coords = [&](int t_local, int& plane, int& tm, int& tn) {
    const int logical = xcd_first + slot_in_xcd + t_local * wgs_per_xcd;
    plane = logical / per_plane;
    const int rem = logical - plane * per_plane;
    tm = rem / tiles_n;
    tn = rem - tm * tiles_n;
  };

  // ---- direct-to-LDS issue.  One instruction = 8 rows x 128 bytes; lane l -> row l/8,
  // LDS chunk' = l%8, global chunk = chunk' ^ key(row).  The key depends on the lane only
  // (and, on the j side, on which 64-row half the row block lies in), so three per-lane byte
  // offsets serve every instruction; everything else is wave-uniform (scalar registers).
  const int lrow = lane >> 3, lchunk = lane & 7;
  const uint32_t off_m0 = (uint32_t)(lrow * row_bytes) + 16u * (lchunk ^ qkey_m<HB>(lrow));
  const uint32_t off_m1 = (uint32_t)(lrow * row_bytes) + 16u * (lchunk ^ qkey_m<HB>(lrow + 64));
  const uint32_t off_n = (uint32_t)(lrow * row_bytes) + 16u * (lchunk ^ qkey_n(lrow));
  const char* dma_base[IPW];  // row-block bases of the tile being loaded (uniform)
  int issue_tile = 0, issue_kb = 0, issue_left = nk, issue_buf = 0;
  auto dma_setup_tile = [&](int t_local) {
    int plane, tm, tn;
    tile_coords(t_local < my_tiles ? t_local : my_tiles - 1, plane, tm, tn);  // past the end: reload the last tile
    const size_t plane_off = (size_t)plane * Np * Np * 2;
    const int rows_m_left = Np - tm * BM, rows_n_left = Np - tn * BN;
#pragma unroll
    for (int n = 0; n < MI; ++n) {
      const int rb = 8 * (wave * MI + n);
      const int rbc = rb + 8 <= rows_m_left ? rb : rows_m_left - 8;  // whole blocks stay inside the plane
      dma_base[n] = reinterpret_cast<const char*>(pm) + plane_off + (size_t)(tm * BM + rbc) * row_bytes;
    }
#pragma unroll
    for (int n = 0; n < NI; ++n) {
      const int rb = 8 * (wave * NI + n);
      const int rbc = rb + 8 <= rows_n_left ? rb : rows_n_left - 8;
      dma_base[MI + n] = reinterpret_cast<const char*>(pn) + plane_off + (size_t)(tn * BN + rbc) * row_bytes;
    }
    issue_kb = (tm + tn) % nk;  // rotated start
    issue_left = nk;
  };
  // one direct-to-LDS instruction of the stage being issued
  auto issue_one = [&](int n) {
    u32x4_t* buf = lds + issue_buf * STAGE;
    const char* src = dma_base[n] + (size_t)issue_kb * (kQBK * 2);
    if (n < MI) {
      const int rb = 8 * (wave * MI + n);
      const uint32_t off = ((rb >> HB) & 1) ? off_m1 : off_m0;
      __builtin_amdgcn_global_load_lds((const void OF3_GLOBAL_AS*)(src + off), (void OF3_LDS_AS*)(buf + rb * 8), 16, 0, 0);
    } else {
      const int rb = 8 * (wave * NI + (n - MI));
      __builtin_amdgcn_global_load_lds((const void OF3_GLOBAL_AS*)(src + off_n), (void OF3_LDS_AS*)(buf + (BM + rb) * 8), 16, 0, 0);
    }
  };
  auto issue_advance = [&]() {
    issue_buf ^= 1;
    issue_kb = issue_kb + 1 == nk ? 0 : issue_kb + 1;
    if (--issue_left == 0) dma_setup_tile(++issue_tile);
  };

  // ---- MFMA operand fetch: k-step ks, lane-half lh reads chunk (2*ks + lh) ^ key
  int am_row[TM], am_key[TM], bn_row[TN], bn_key[TN];
  {
    const int g = l32 >> 3, hb = (l32 >> 2) & 1, e = l32 & 3;
#pragma unroll
    for (int mt = 0; mt < TM; ++mt) {
      const int row = wm0 + 16 * TM * hb + 16 * mt + 4 * g + e;
      am_row[mt] = row * 8;
      am_key[mt] = qkey_m<HB>(row) ^ lh;
    }
#pragma unroll
    for (int nt = 0; nt < TN; ++nt) {
      const int row = wn0 + 32 * nt + l32;
      bn_row[nt] = (BM + row) * 8;
      bn_key[nt] = qkey_n(row) ^ lh;
    }
  }
  auto fetch = [&](const u32x4_t* buf, int ks, u32x4_t (&af)[TM], u32x4_t (&bfr)[TN]) {
#pragma unroll
    for (int mt = 0; mt < TM; ++mt) af[mt] = buf[am_row[mt] + ((2 * ks) ^ am_key[mt])];
#pragma unroll
    for (int nt = 0; nt < TN; ++nt) bfr[nt] = buf[bn_row[nt] + ((2 * ks) ^ bn_key[nt])];
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
  // the same, with the stage's loads issued in between (two per MFMA until they run out)
  auto mma_and_issue = [&](const u32x4_t (&af)[TM], const u32x4_t (&bfr)[TN]) {
    int n = 0;
#pragma unroll
    for (int mt = 0; mt < TM; ++mt)
#pragma unroll
      for (int nt = 0; nt < TN; ++nt) {
        acc[mt][nt] = mfma_32x32x16(af[mt], bfr[nt], acc[mt][nt]);
        if (n < IPW) issue_one(n++);
        if (n < IPW) issue_one(n++);
      }
    issue_advance();
  };

  // ---- prologue: two stages in flight, the first one visible
  dma_setup_tile(0);
#pragma unroll
  for (int n = 0; n < IPW; ++n) issue_one(n);
  issue_advance();
#pragma unroll
  for (int n = 0; n < IPW; ++n) issue_one(n);
  issue_advance();
  wait_vmcnt<IPW>();
  compiler_fence();
  __builtin_amdgcn_s_barrier();
  compiler_fence();

  u32x4_t a0[TM], b0[TN], a1[TM], b1[TN];
  fetch(lds, 0, a0, b0);

  int cur_buf = 0;
  bool stores_pending = false;  // the previous tile's full set of output stores is still in the queue
  for (int t_local = 0; t_local < my_tiles; ++t_local) {
    for (int kb = 0; kb < nk; ++kb) {
      const u32x4_t* cur = lds + cur_buf * STAGE;
      fetch(cur, 1, a1, b1);
      mma(a0, b0);
      fetch(cur, 2, a0, b0);
      mma(a1, b1);
      fetch(cur, 3, a1, b1);
      mma(a0, b0);
      __builtin_amdgcn_sched_barrier(0);

      // All of this stage is in registers now; the next stage (issued one stage ago) must
      // have landed.  VMEM operations retire in order; the queue holds, oldest first,
      // [next stage's loads][output stores of the tile that has just ended, if any], so
      // those stores may stay outstanding.
      __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
      if (stores_pending) wait_vmcnt<8 * TN>();
      else wait_vmcnt<0>();
      stores_pending = false;
      compiler_fence();
      __builtin_amdgcn_s_barrier();
      compiler_fence();
      __builtin_amdgcn_sched_barrier(0);

      cur_buf ^= 1;
      fetch(lds + cur_buf * STAGE, 0, a0, b0);  // past the last stage this reads stale data that is never used
      mma_and_issue(a1, b1);                    // refills the buffer this stage has just left
      __builtin_amdgcn_sched_barrier(0);
    }

    // ---- tile finished.  Each wave transposes its 32-row blocks through a private 8 KB
    // LDS region (row-major [32 i][128 j] bf16, 16-byte chunks XOR-swizzled by the row) and
    // writes whole 256-byte row segments.
    int plane, tm, tn;
    tile_coords(t_local, plane, tm, tn);
    bf16_t* xo = x + (size_t)plane * Np * Np;
    u32x4_t* epi = lds + 2 * STAGE + wave * 512;
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
        const int chunk = 8 * lh + 2 * mt;
        epi[l32 * 16 + (chunk ^ (l32 & 7))] = lo;
        epi[l32 * 16 + ((chunk + 1) ^ (l32 & 7))] = hi;
        acc[mt][nt] = zero16();
      }
      const int i0 = tn * BN + wn0 + 32 * nt;
      if (i0 < Np && jbase < Np) {  // wave-uniform: Np is a multiple of 128
#pragma unroll
        for (int rr = 0; rr < 8; ++rr) {
          const int row = 4 * rr + (lane >> 4), chunk = lane & 15;
          const u32x4_t v = epi[row * 16 + (chunk ^ (row & 7))];
          *reinterpret_cast<u32x4_t*>(xo + (size_t)(i0 + row) * Np + jbase + 8 * chunk) = v;
        }
        n_stores += 8;
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    // only a complete set of stores is accounted for exactly; otherwise the next wait
    // simply covers them too (waiting for more than necessary is always safe)
    stores_pending = (n_stores == 8 * TN);
  }
  wait_vmcnt<0>();  // the loads issued past the end must not outlive the work-group's LDS
}

template <int BM, int BN>
hipError_t launch_pipe64(const bf16_t* a, const bf16_t* b, bf16_t* x, int planes, int Np, hipStream_t stream) {
  auto kern = contract_pipe64_kernel<BM, BN>;
  const size_t smem = ((size_t)2 * (BM + BN) * 8 + 4 * 512) * sizeof(u32x4_t);
  static int cus = 0;
  if (cus == 0) {
    int dev = 0, n = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    e = hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev);
    if (e != hipSuccess) return e;
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)smem);
    if (e != hipSuccess) return e;
    cus = n;
  }
  const int tiles_m = (Np + BM - 1) / BM, tiles_n = (Np + BN - 1) / BN;
  const int total = planes * tiles_m * tiles_n;
  const int tiles_per_xcd = (total + 7) / 8;
  int grid = (cus / 8) * 8;
  if (grid < 8) grid = 8;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(256), smem, stream, b, a, x, Np, tiles_m, tiles_n, total, tiles_per_xcd);
  return hipGetLastError();
}

template <int BM, int BN>
hipError_t launch_pipe(const bf16_t* a, const bf16_t* b, bf16_t* x, int planes, int Np, hipStream_t stream) {
  auto kern = contract_pipe_kernel<BM, BN>;
  const size_t smem = ((size_t)kNS * (BM + BN) * 4 + 4 * 512) * sizeof(u32x4_t);  // ring + epilogue staging
  static int cus = 0;
  if (cus == 0) {
    int dev = 0, n = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    e = hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev);
    if (e != hipSuccess) return e;
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)smem);
    if (e != hipSuccess) return e;
    cus = n;
  }
  const int tiles_m = (Np + BM - 1) / BM, tiles_n = (Np + BN - 1) / BN;
  const int total = planes * tiles_m * tiles_n;
  const int tiles_per_xcd = (total + 7) / 8;
  int grid = (cus / 8) * 8;  // a multiple of the 8 XCDs
  if (grid < 8) grid = 8;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(256), smem, stream, b, a, x, Np, tiles_m, tiles_n, total, tiles_per_xcd);
  return hipGetLastError();
}

}  // namespace

hipError_t trimul_contract_pipe_launch(const bf16_t* a, const bf16_t* b, bf16_t* x, int planes, int Np, int variant,
                                       hipStream_t stream) {
  switch (variant) {
    case 4:
      return launch_pipe<256, 192>(a, b, x, planes, Np, stream);
    case 5:
      return launch_pipe<256, 256>(a, b, x, planes, Np, stream);
    case 6:
      return launch_pipe<256, 128>(a, b, x, planes, Np, stream);
    case 7:
      return launch_pipe64<256, 192>(a, b, x, planes, Np, stream);
    default:
      return hipErrorInvalidValue;
  }
}

}  // namespace of3

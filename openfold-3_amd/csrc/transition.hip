// Pair transition (SwiGLUTransition, transition.py:225-271 with SwiGLU of activations.py:33-61,
// and the caller's residual add of base_blocks.py:470-478 when requested):
//     out = [x +] ((silu(xn Wa^T) * (xn Wb^T)) Wout^T) * mask,   xn = LayerNorm(x)
// Position-wise, 6*C*HID flops per position (HID = n*C), i.e. MFMA bound: both GEMMs are chained
// in registers, nothing but x and out touches HBM.
//
// Organisation:
//  * work-group = 8 waves, a tile = 256 consecutive positions of one row; a wave owns 32
//    positions.  Their normalised activations are staged once through a wave-private LDS tile
//    and then held in registers as MFMA B operands for the whole tile.
//  * the hidden dimension is walked in tiles of 32 channels.  The weights of a hidden tile (32
//    rows of Wa and of Wb, 32 columns of Wout) are shared by all waves and travel
//    L2 -> LDS with direct-to-LDS loads, two hidden tiles ahead (one vmcnt wait + one barrier
//    per hidden tile), through a 3-deep ring for Wa/Wb and a 4-deep one for Wout; the rings
//    run on across tiles, the sequence of hidden tiles simply repeats.
//  * per hidden tile: a^T, b^T = W{a,b}[32 x C] * xn^T (A from LDS, B from registers), then
//    h = silu(a) * b in fp32, rounded to bf16, is already laid out as the B operand of the
//    second product (a lane holds 16 consecutive hidden channels of its position), so
//    out^T += Wout[C x 32] * h^T needs no data movement between the two GEMMs.
//  * software pipeline: the SiLU arithmetic of hidden tile t-1 (vector ALU, two
//    transcendentals per element) is interleaved, element by element, with the first
//    product's MFMAs of tile t, and the second product of tile t-1 follows; a wave issues in
//    order, so without this its matrix and vector phases (about equally long) add up instead
//    of overlapping.  That is why Wout stays one step longer in LDS than Wa/Wb.
//  * epilogue: mask and residual (the activations as loaded wait in the wave's LDS tile during
//    the hidden loop) in the accumulator layout, transposed through that tile, whole rows
//    stored, next tile's loads issued.
//    Positions past the end of a row are treated as copies of the last one (indices clamped:
//    they load, compute and store the same bytes), so every tile issues the same sequence of
//    memory instructions and the waits on the in-order memory counter are static.
#include <type_traits>

#include "of3_device.h"
#include "of3_kernels.h"
#include "of3_launch.h"

namespace of3 {

namespace {

#define OF3_GLOBAL_AS __attribute__((address_space(1)))
#define OF3_LDS_AS __attribute__((address_space(3)))

constexpr int kWaves = 8;
constexpr int kStagesW = 3;  // Wa/Wb ring: a stage is read in its own step
constexpr int kStagesO = 4;  // Wout ring: a stage is read in the step after its own
constexpr int kPD = 2;       // prefetch distance in hidden tiles

__device__ __forceinline__ void compiler_fence() { __asm__ volatile("" ::: "memory"); }
template <int N>
__device__ __forceinline__ void wait_vmcnt() {  // vmcnt(N) only (gfx9 encoding, 6-bit counter)
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
  __builtin_amdgcn_s_waitcnt((N & 15) | 0x70 | 0xF00 | ((N >> 4) << 14));
}

// Swizzle keys.  A ds_read_b128 is served 16 lanes (256 bytes, all 64 banks) per cycle; the 16
// lanes of an MFMA A-operand read hold rows {0..7, 16..23} or {8..15, 24..31} of a tile
// (rowperm16) at one chunk index, so the key must spread those rows over one 256-byte window.
template <int NCH>
__device__ __forceinline__ int key_w(int row) {  // Wa / Wb tile rows of NCH chunks
  return NCH == 16 ? (row & 7) | ((row >> 1) & 8)            // one row per window: 16 distinct keys
                   : ((row >> 1) & 3) | ((row >> 2) & 4);    // two rows per window: 8 keys per row parity
}
template <int NCH>
__device__ __forceinline__ int key_x(int pos) {  // wave-private activation tile, 32 positions of NCH chunks
  return NCH == 16 ? pos & 15 : (pos >> 1) & 7;  // B-operand reads: 16 consecutive positions at one chunk index
}
__device__ __forceinline__ int key_o(int row) {                                         // Wout tile rows (64 B)
  return ((((row >> 4) ^ (row >> 1)) & 1) << 1) | (((row >> 2) ^ (row >> 1)) & 1);
}

template <int C>
__global__ __launch_bounds__(64 * kWaves) void transition_kernel(TransitionArgs p, int tiles_per_row, int total_tiles) {
  constexpr int NCH = C / 8;             // 16-byte chunks per position / per W{a,b} row
  constexpr int PPI = 64 / NCH;          // positions per wave instruction in the row-wise phases
  constexpr int ROWS = 32;               // positions per wave
  constexpr int ITERS = ROWS / PPI;      // row-wise instructions per wave and tile
  constexpr int KS = C / 16;             // k-steps of the first product
  constexpr int CT = C / 32;             // output-channel tiles of the second product
  constexpr int WSLOTS = 32 * NCH;       // one Wa (or Wb) hidden tile
  constexpr int OSLOTS = C * 4;          // one Wout hidden tile: C rows x 64 bytes
  constexpr int STAGE = 2 * WSLOTS + OSLOTS;
  constexpr int DMA_TOTAL = STAGE / 64;  // direct-to-LDS instructions per stage (24 or 12)
  constexpr int LPT = (DMA_TOTAL + kWaves - 1) / kWaves;  // per wave; surplus slots re-load a piece twice
  constexpr int NLD = ITERS + 1;         // loads of a tile: activations and mask
  static_assert(LPT + NLD + ITERS < 64, "vmcnt budget");

  extern __shared__ u32x4_t lds[];
  u32x4_t* ring_w = lds;                                   // [kStagesW][2 * WSLOTS]
  u32x4_t* ring_o = lds + kStagesW * 2 * WSLOTS;           // [kStagesO][OSLOTS]
  u32x4_t* mine = ring_o + kStagesO * OSLOTS + (threadIdx.x >> 6) * (ROWS * NCH);  // wave-private [32 pos][NCH]

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63, l32 = lane & 31, lh = lane >> 5;
  const int rw_chunk = lane % NCH, rw_pp = lane / NCH;  // row-wise phases: 16 bytes of one position per lane
  const int N = p.N, NHT = p.HID / 32;

  // LayerNorm parameters of this lane's chunk, kept packed (8 registers) between tiles
  u32x4_t lw_pk = *reinterpret_cast<const u32x4_t*>(p.ln_w + 8 * rw_chunk);
  u32x4_t lb_pk = *reinterpret_cast<const u32x4_t*>(p.ln_b + 8 * rw_chunk);

  // ---- direct-to-LDS sources of this wave's LPT instructions (byte offsets inside hidden tile 0;
  // a hidden tile further on adds a wave-uniform offset).  Instruction q covers slots
  // 64q .. 64q+63 of the stage: first the Wa tile, then Wb (one ring), then Wout (the other).
  uint32_t dma_off[LPT];
  const char* dma_base[LPT];  // wave-uniform
  int dma_step[LPT], dma_slot[LPT];
  bool dma_out[LPT];
#pragma unroll
  for (int n = 0; n < LPT; ++n) {
    const int q = (LPT * wave + n) % DMA_TOTAL;
    const int t = 64 * q + lane;
    dma_out[n] = 64 * q >= 2 * WSLOTS;
    dma_slot[n] = dma_out[n] ? 64 * q - 2 * WSLOTS : 64 * q;
    if (!dma_out[n]) {  // Wa or Wb: slot (row, c') holds chunk c' ^ key_w(row) of row `row` of the tile
      const int tt = t % WSLOTS, row = tt / NCH, chunk = (tt % NCH) ^ key_w<NCH>(row);
      dma_base[n] = reinterpret_cast<const char*>(64 * q < WSLOTS ? p.w_a : p.w_b);
      dma_step[n] = 32 * C * (int)sizeof(bf16_t);
      dma_off[n] = (uint32_t)((row * C + 8 * chunk) * sizeof(bf16_t));
    } else {                    // Wout: slot (row, c') holds chunk c' ^ key_o(row) of the 64-byte piece of row `row`
      const int tt = t - 2 * WSLOTS, row = tt >> 2, chunk = (tt & 3) ^ key_o(row);
      dma_base[n] = reinterpret_cast<const char*>(p.w_out);
      dma_step[n] = 32 * (int)sizeof(bf16_t);
      dma_off[n] = (uint32_t)((row * p.HID + 8 * chunk) * sizeof(bf16_t));
    }
  }
  auto issue_stage = [&](int ht, int buf_w, int buf_o) {
#pragma unroll
    for (int n = 0; n < LPT; ++n) {
      const char* src = dma_base[n] + (size_t)ht * dma_step[n] + dma_off[n];
      u32x4_t* dst = (dma_out[n] ? ring_o + buf_o * OSLOTS : ring_w + buf_w * 2 * WSLOTS) + dma_slot[n];
      __builtin_amdgcn_global_load_lds((const void OF3_GLOBAL_AS*)src, (void OF3_LDS_AS*)dst, 16, 0, 0);
    }
  };

  // ---- operand read slots
  const int arow = rowperm16(l32);  // A rows are dealt so that a lane ends with 16 consecutive output rows
  // W{a,b}: chunk 2s+lh of row arow
  int wa_rd[KS];
#pragma unroll
  for (int s = 0; s < KS; ++s) wa_rd[s] = arow * NCH + ((2 * s + lh) ^ key_w<NCH>(arow));
  // Wout: k-step s, lane-half lh <-> hidden 16*lh + 8*s + (0..7) = chunk 2*lh + s of row
  // 32*ct + arow; the key does not depend on ct.
  int wo_rd2[2];
#pragma unroll
  for (int s = 0; s < 2; ++s) wo_rd2[s] = arow * 4 + ((2 * lh + s) ^ key_o(arow));

  // ---- tile bookkeeping
  const int tiles_per_batch = p.R * tiles_per_row;
  u32x4_t raw[ITERS];
  float mval;
  auto tile_row = [&](int tile_id, int& j0) {
    const int b = tile_id / tiles_per_batch;
    const int rem = tile_id - b * tiles_per_batch;
    const int i = rem / tiles_per_row;
    j0 = (rem - i * tiles_per_row) * (ROWS * kWaves) + ROWS * wave;
    return (int64_t)b * p.x_view.stride_b + (int64_t)i * p.x_view.stride_r;
  };
  // Element offsets along a row fit 32 bits (checked by the launcher), so a row is a uniform
  // base pointer plus a 32-bit lane offset.
  const uint32_t sk_bytes = (uint32_t)p.x_view.stride_k * (uint32_t)sizeof(bf16_t);
  const uint32_t mk_bytes = (uint32_t)p.mask_view.stride_k * (uint32_t)sizeof(float);
  auto load_tile = [&](int tile_id) {
    int j0;
    const char* xrow = reinterpret_cast<const char*>(p.x + tile_row(tile_id, j0));
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      int j = j0 + it * PPI + rw_pp;
      j = j < N ? j : N - 1;
      raw[it] = *reinterpret_cast<const u32x4_t*>(xrow + ((uint32_t)j * sk_bytes + 16u * rw_chunk));
    }
    // mask of the position this lane owns in the MFMA phases; without a mask the load still
    // happens (from the LayerNorm weights) so that the instruction count does not depend on it
    int j = j0 + l32;
    j = j < N ? j : N - 1;
    const int b = tile_id / tiles_per_batch;
    const int i = (tile_id - b * tiles_per_batch) / tiles_per_row;
    const char* mrow = p.mask ? reinterpret_cast<const char*>(p.mask + (int64_t)b * p.mask_view.stride_b +
                                                              (int64_t)i * p.mask_view.stride_r)
                              : reinterpret_cast<const char*>(p.ln_w);
    mval = *reinterpret_cast<const float*>(mrow + (p.mask ? (uint32_t)j * mk_bytes : 0u));
  };

  const int my_tiles = (int)blockIdx.x < total_tiles ? (total_tiles - (int)blockIdx.x + (int)gridDim.x - 1) / (int)gridDim.x : 0;
  if (my_tiles == 0) return;

  load_tile(blockIdx.x);
  // Stages are requested unconditionally, two more than are consumed at the very end (they
  // land in buffers nobody reads again): the number of memory instructions between any two
  // points of the program is then fixed, which is what the waits below rely on.
  int issue_ht = 0;  // hidden tile of the next stage to request
  int issue_w = 0, issue_o = 0;
  auto issue_next = [&]() {
    issue_stage(issue_ht, issue_w, issue_o);
    issue_ht = issue_ht + 1 == NHT ? 0 : issue_ht + 1;
    issue_w = issue_w + 1 == kStagesW ? 0 : issue_w + 1;
    issue_o = issue_o + 1 == kStagesO ? 0 : issue_o + 1;
  };
#pragma unroll
  for (int s = 0; s < kPD; ++s) issue_next();

  // ---- LayerNorm -> wave-private LDS tile -> B operands in registers, for the tile whose
  // activations are in `raw`.  Runs before the first tile and at the end of every tile for
  // the next one, before that tile's stores are issued (see there).
  u32x4_t xb[KS];
  float mtile;
  auto prepare_tile = [&]() {
    // lane-derived slot numbers of this phase are recomputed every time (a few instructions)
    // instead of living in registers through the hidden loop
    int lane_t = lane;
    __asm__ volatile("" : "+v"(lane_t));
    const int t_chunk = lane_t % NCH, t_pp = lane_t / NCH, t_l32 = lane_t & 31, t_lh = lane_t >> 5;
    u32x4_t tw = lw_pk, tb = lb_pk;
    __asm__ volatile("" : "+v"(tw), "+v"(tb));  // unpacked here rather than held as 16 floats
    float lw[8], lb[8];
    unpack8(tw, lw);
    unpack8(tb, lb);
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      const int pos = it * PPI + t_pp;
      mine[pos * NCH + (t_chunk ^ key_x<NCH>(pos))] = layer_norm_chunk<C>(raw[it], lw, lb);
    }
#pragma unroll
    for (int s = 0; s < KS; ++s) xb[s] = mine[t_l32 * NCH + ((2 * s + t_lh) ^ key_x<NCH>(t_l32))];
    // the tile then keeps the activations as loaded: the residual of the epilogue
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      const int pos = it * PPI + t_pp;
      mine[pos * NCH + (t_chunk ^ key_x<NCH>(pos))] = raw[it];
    }
    mtile = p.mask ? mval : 1.f;
  };
  prepare_tile();

  int buf_w = 0, buf_o = 0;  // buffers of the stage the next step consumes
  for (int tl = 0; tl < my_tiles; ++tl) {
    const int tile_id = blockIdx.x + tl * gridDim.x;
    int j0;
    const int64_t row_off = tile_row(tile_id, j0);

    f32x16_t oacc[CT];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) oacc[ct] = zero16();
    f32x16_t pa, pb;  // a^T, b^T of the previous hidden tile, waiting for their SiLU and second product
    u32x4_t hb[2];    // h of that tile as bf16: lane-half lh, register v = hidden 16*lh + v

    // element e of h = silu(a) * b from the previous hidden tile's a, b
    auto silu_elem = [&](int e) {
      const float h = pa[e] * fast_rcp(1.f + fast_exp2(-kLog2e * pa[e])) * pb[e];
      pa[e] = h;
      if (e & 1) hb[e >> 3][(e & 7) >> 1] = pack_bf16(pa[e - 1], h);
    };
    // out^T += Wout[:, previous hidden tile] * h^T, Wout from ring buffer `bo`
    auto second_product = [&](const u32x4_t* so) {
      u32x4_t oq[4];
#pragma unroll
      for (int i = 0; i < 4 && i < 2 * CT; ++i) oq[i] = so[wo_rd2[i / CT] + 128 * (i % CT)];
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < 2 * CT; ++i) {
        oacc[i % CT] = mfma_32x32x16(oq[i & 3], hb[i / CT], oacc[i % CT]);
        if (i + 4 < 2 * CT) oq[i & 3] = so[wo_rd2[(i + 4) / CT] + 128 * ((i + 4) % CT)];
        __builtin_amdgcn_sched_barrier(0);
      }
    };

    // One hidden tile.  KIND 0: the first of a tile (nothing to finish from the previous
    // one); 1: any other but the last two; 2: the last but one, which also issues the next
    // tile's loads; 3: the last.
    auto hidden_step = [&](int ht, auto kind_tag) {
      constexpr int KIND = decltype(kind_tag)::value;
      // Stage `ht` must have landed.  Memory operations retire in issue order, so "at most
      // n outstanding" means everything older than the newest n is complete.  Younger than
      // the stage: the next stage and whatever else was issued since the request two steps
      // ago: the next tile's NLD loads (issued in the last step but one of every tile) and
      // the ITERS stores of the previous tile's epilogue.
      if (KIND == 3) wait_vmcnt<LPT + NLD>();
      else if (KIND == 0 && tl > 0) wait_vmcnt<LPT + NLD + ITERS>();
      else if (KIND == 1 && tl > 0 && ht == 1) wait_vmcnt<LPT + ITERS>();
      else wait_vmcnt<LPT>();
      __builtin_amdgcn_s_barrier();  // everybody's part of the stage is visible; the buffers that
      compiler_fence();              // the stage two ahead goes into are no longer read
      issue_next();
      // next tile's activations, early enough to arrive under the last two hidden tiles (a
      // dummy reload of this tile after the last one keeps the instruction count per tile fixed)
      if (KIND == 2) load_tile(tl + 1 < my_tiles ? tile_id + gridDim.x : tile_id);
      const u32x4_t* sw = ring_w + buf_w * 2 * WSLOTS;
      const u32x4_t* so_prev = ring_o + (buf_o == 0 ? kStagesO - 1 : buf_o - 1) * OSLOTS;
      buf_w = buf_w + 1 == kStagesW ? 0 : buf_w + 1;
      buf_o = buf_o + 1 == kStagesO ? 0 : buf_o + 1;

      // ---- a^T, b^T of this hidden tile (32 hidden rows x this wave's 32 positions): the
      // 2*KS A operands (Wa k-steps, then Wb) pass through a four-deep register ring, four
      // reads ahead of their MFMA; each MFMA is followed by the SiLU arithmetic of 16/(2*KS)
      // elements of the previous tile.  The source order is the issue order (scheduling fences).
      constexpr int EPS = 16 / (2 * KS);
      auto w_op = [&](int i) -> u32x4_t {
        return sw[(i < KS ? 0 : WSLOTS) + wa_rd[i % KS]];
      };
      f32x16_t ca = zero16(), cb = zero16();
      u32x4_t aq[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) aq[i] = w_op(i);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < 2 * KS; ++i) {
        if (i < KS) ca = mfma_32x32x16(aq[i & 3], xb[i], ca);
        else cb = mfma_32x32x16(aq[i & 3], xb[i - KS], cb);
        if (i + 4 < 2 * KS) aq[i & 3] = w_op(i + 4);
        if (KIND != 0) {
#pragma unroll
          for (int e = EPS * i; e < EPS * (i + 1); ++e) silu_elem(e);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      if (KIND != 0) second_product(so_prev);
      pa = ca;
      pb = cb;
    };
    hidden_step(0, std::integral_constant<int, 0>{});
    for (int ht = 1; ht < NHT - 2; ++ht) hidden_step(ht, std::integral_constant<int, 1>{});
    hidden_step(NHT - 2, std::integral_constant<int, 2>{});
    hidden_step(NHT - 1, std::integral_constant<int, 3>{});
    // the last hidden tile's SiLU and second product (its Wout stays valid until two barriers on)
#pragma unroll
    for (int e = 0; e < 16; ++e) silu_elem(e);
    second_product(ring_o + (buf_o == 0 ? kStagesO - 1 : buf_o - 1) * OSLOTS);

    char* orow = reinterpret_cast<char*>(p.out + row_off);
    // ---- epilogue: mask, residual (read from the wave's LDS tile in the accumulator layout and
    // replaced in place by the result), then whole rows leave through the row-wise mapping
    int lane_e = lane;
    __asm__ volatile("" : "+v"(lane_e));
    const int e_chunk = lane_e % NCH, e_pp = lane_e / NCH, e_l32 = lane_e & 31, e_lh = lane_e >> 5;
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
      const int chunk = 4 * ct + 2 * e_lh;  // channels 32*ct + 16*lh + (0..15)
      const int s0 = e_l32 * NCH + (chunk ^ key_x<NCH>(e_l32));
      const int s1 = e_l32 * NCH + ((chunk + 1) ^ key_x<NCH>(e_l32));
      float r0[8], r1[8];
      unpack8(mine[s0], r0);
      unpack8(mine[s1], r1);
      if (!p.add_residual) {
#pragma unroll
        for (int e = 0; e < 8; ++e) r0[e] = r1[e] = 0.f;
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        r0[e] += oacc[ct][e] * mtile;
        r1[e] += oacc[ct][8 + e] * mtile;
      }
      mine[s0] = pack8(r0);
      mine[s1] = pack8(r1);
    }
    u32x4_t outv[ITERS];
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      const int pos = it * PPI + e_pp;
      outv[it] = mine[pos * NCH + (e_chunk ^ key_x<NCH>(pos))];
    }
    // The next tile is prepared before this tile's stores are issued: direct-to-LDS loads in
    // flight make the compiler wait for every outstanding memory operation at the first use
    // of a loaded register, and here the only young ones are the stage requests.  (After the
    // last tile this processes the dummy reload: unconditional, so that no path leaves the
    // loaded registers pending.)
    prepare_tile();
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      int j = j0 + it * PPI + e_pp;
      j = j < N ? j : N - 1;  // copies of the last position store the same bytes
      *reinterpret_cast<u32x4_t*>(orow + ((uint32_t)j * sk_bytes + 16u * e_chunk)) = outv[it];
    }
  }
  wait_vmcnt<0>();
}

template <int C>
hipError_t launch(const TransitionArgs& a, hipStream_t stream) {
  auto kern = transition_kernel<C>;
  constexpr int smem = (kStagesW * 2 * 32 * (C / 8) + kStagesO * C * 4 + kWaves * 32 * (C / 8)) * 16;
  static int cache[kMaxDevices];
  int cus = 0;
  hipError_t e = per_device(
      cache,
      [&](int dev, int* v) {
        hipError_t s = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, smem);
        return s != hipSuccess ? s : cu_count(dev, v);
      },
      &cus);
  if (e != hipSuccess) return e;
  if ((uint64_t)(a.N - 1) * (uint64_t)a.x_view.stride_k * 2 + 2 * C > 0xffffffffull ||
      (a.mask && (uint64_t)(a.N - 1) * (uint64_t)a.mask_view.stride_k * 4 + 4 > 0xffffffffull))
    return hipErrorInvalidValue;
  const int tiles_per_row = (a.N + 32 * kWaves - 1) / (32 * kWaves);
  if (a.R < 1) return hipErrorInvalidValue;
  const long total = (long)a.B * a.R * tiles_per_row;
  if (total > 0x7fffffffl) return hipErrorInvalidValue;
  const int grid = (int)(total < cus ? total : cus);
  hipLaunchKernelGGL(kern, dim3(grid), dim3(64 * kWaves), smem, stream, a, tiles_per_row, (int)total);
  return hipGetLastError();
}

}  // namespace

hipError_t transition_launch(const TransitionArgs& args, int C, hipStream_t stream) {
  if (args.HID % 32 != 0 || args.HID < 128) return hipErrorInvalidValue;  // at least four hidden tiles
  if (C == 128) return launch<128>(args, stream);
  if (C == 64) return launch<64>(args, stream);
  return hipErrorInvalidValue;
}

}  // namespace of3

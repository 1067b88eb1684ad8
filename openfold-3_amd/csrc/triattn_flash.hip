// Triangle-attention core (attention.py:94-135 with the two biases of tri_att.py:134-140):
//     s[q][k] = q.k + mb[i][k] + tb[h][q][k];  p = softmax_k(s);  o[q] = sum_k p[q][k] v[k]
// for every (batch, row i, head h), flash style: 32-key tiles, fp32 row sums, no [N][N] logits in
// memory.  Inputs come from the projection pass already multiplied by log2(e) (q also by
// 1/sqrt(D)), so exp() is the hardware exp2.
//
// With head width 16 or 32 the kernel is bound by the softmax's vector instructions (a SIMD spends
// matrix time plus vector time), so the organisation removes vector work and keeps four waves per
// SIMD to cover each other's waits:
//  * work-group = 8 waves = 4 consecutive rows i x 2 halves of one (head, 128-query range); a wave
//    owns 64 queries (two 32-query tiles) of one row; two work-groups share a CU (64 KB of LDS and
//    128 registers per lane each).  The triangle bias of the query range does not depend on i:
//    each 32-key slice of it is brought into LDS once per work-group and every wave reads it
//    straight into the MFMA accumulator, which adds it for free.
//  * everything a key tile needs (the work-group's bias slice, each row's K tile and V^T tile,
//    loaded by one wave of the row each) travels global -> LDS with direct-to-LDS buffer loads, one
//    tile ahead, into double buffers; the only wait is one vmcnt(0) + barrier per key tile, a whole
//    tile of arithmetic after the loads were issued.  The XOR swizzles are applied on the global
//    side (a lane picks which 16-byte chunk it fetches for its fixed LDS slot).
//  * S^T = K Q^T: A = K tile (row r of the tile is key rowperm16(r), so a lane ends up with
//    16 consecutive keys of one query), B = Q tile (registers).  O^T = V^T P^T: A = V^T,
//    B = P^T taken directly from the S^T accumulator registers (no cross-lane movement).
//  * the first pass over the keys uses the offset 0 for every query: a logit costs one exp2, one
//    add and half a pack, no maximum and no subtraction.  Any common offset gives the same
//    softmax; whether 0 was good enough is read off the row sum at the end (within 2^-60..2^60),
//    and a work-group with a query outside that range (overflow, a row of masked keys) repeats
//    the pass with running maxima: raised only when a logit exceeds the offset by 2^64, snapped
//    to 0 when within +-32, subtracted exactly by one more MFMA k-step.
//  * the mask bias of a key tile rides on one more k-step of the S^T product (A = [mb[key],
//    0, ...], B = [1, 0, ...]) right after the triangle bias, i.e. (tb + mb) + q.k in the
//    fp32 accumulator: masked keys get weight exactly 0, padded keys (N not a multiple of
//    32) carry -inf, and a fully masked row degenerates to a uniform average over all real
//    keys exactly as the reference's does (-1e9 absorbs the logits in fp32).  A key tile whose
//    32 mask biases are all zero (checked wave-wide once per tile) skips that k-step.
//  * padding costs no arithmetic in the first pass: a key tile whose 32 keys are all masked or padded
//    contributes exp2(-1.44e9 + logit) = 0 exactly to every sum, so the wave leaves that tile out (its
//    loads and barriers go on).  A row without any unmasked key (a padded token) thereby sits the first
//    pass out, ends it with the row sum 0 and takes the pass with running maxima, which gives the
//    reference's uniform average (padded tokens come in runs, so the four rows of a work-group mostly
//    agree and few other rows are dragged into a second pass).
//  * head width 16 leaves rows 16..31 of the V^T operand free: row 16 holds ones, so the PV product
//    itself accumulates the row sum (of the bf16 weights it multiplies) and the 16 additions per tile go.
#include "of3_device.h"
#include "of3_kernels.h"
#include "of3_launch.h"

#include <type_traits>

// Token count from which the 16-wave form (256 queries per work-group, one work-group per CU) is used.
// Measured against the 8-wave form (two work-groups per CU): N = 768 395 vs 375 us, N = 2048 7.57 vs
// 6.95 ms, 4 x 512 with head width 16 474 vs 400 us: the K / V^T loads it saves cost less than the second
// independent work-group hides, so the default is never.
#ifndef OF3_FLASH_WIDE_FROM
#define OF3_FLASH_WIDE_FROM (1 << 30)
#endif

namespace of3 {

namespace {

__device__ __forceinline__ float xhalf(float v) { return __shfl_xor(v, 32, 64); }

typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4_t;
__device__ __forceinline__ f32x4_t mfma_16x16x32(u32x4_t a, u32x4_t b, f32x4_t c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
}

// swizzle keys of the K / V^T tiles in LDS: rows are read in the order rowperm16(lane), i.e.
// {x..x+3, x+16..x+19, x+4..x+7, x+20..x+23} per 16 lanes; (row & 1, key) must differ inside
// every group of 8 lanes and (row & 3, key) inside every group of 16
__device__ __forceinline__ int key4(int row) {  // 4 chunks (64 bytes) per row
  return ((((row >> 4) ^ (row >> 1)) & 1) << 1) | (((row >> 2) ^ (row >> 1)) & 1);
}
__device__ __forceinline__ int key2(int row) { return (row >> 4) & 1; }  // 2 chunks per row

// Every iteration of the tile loop issues the same loads (indices past the end are clamped, their
// data is never read), so that the compiler can count the loads in flight and its own waits do not
// drain the ring.
// 32-query tiles per wave: 2 (the shipped form) or 1 (half the accumulators, so that six waves per SIMD fit:
// measured slower, head width 16 at 4 x 512^2 443 vs 392 us with 76 registers and no spills, head width 32
// does not fit 80 registers; a K / V^T tile read from LDS then serves half as many logits)
#ifndef OF3_FLASH_RQ
#define OF3_FLASH_RQ 2
#endif
constexpr int kRows = 4, kRQ = OF3_FLASH_RQ, kStages = 2;
constexpr int kQW = 32 * kRQ;  // queries per wave
#ifndef OF3_FLASH_RG_BLOCK
#define OF3_FLASH_RG_BLOCK 8
#endif
constexpr int kRgBlock = OF3_FLASH_RG_BLOCK, kQcBlock = 8;  // row groups x query ranges per block of the work-group order
constexpr float kRaise = 64.0f;  // the offset of a query is raised only when a logit exceeds it by 2^64 ...
constexpr float kSnap = 32.0f;   // ... and an offset within +-32 is replaced by 0
constexpr float kMaskedBelow = -1e8f;  // a mask bias below this sends exp2 of any sane logit to exactly 0

__device__ __forceinline__ float max3(float a, float b, float c) {
  float r;
  __asm__("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}

// QW = waves per row: 2 (work-group = 8 waves = 4 rows x 128 queries, two work-groups per CU) or 4 (16 waves
// = 4 rows x 256 queries, one work-group per CU: a row's K and V^T tiles, the loads that miss L2, are brought
// in for twice as many queries).
template <int D, int QW>
__global__ __launch_bounds__(64 * kRows * QW, kRQ == 1 ? 6 : 4) void triattn_flash_kernel(TriattnFlashArgs p, int n_qc, int n_rg,
                                                                             int total, int per_xcd) {
  constexpr int kWaves = kRows * QW;
  constexpr int QWG = kQW * QW;  // queries per work-group
  constexpr int H = 4;
  constexpr int HD = H * D;
  constexpr int KSQ = D / 16;
  constexpr int QCH = D / 8;
  constexpr int KSLOTS = 32 * QCH;
  constexpr int VSLOTS = D * 4;
  constexpr int KVS = KSLOTS + VSLOTS;
  constexpr int KI = KSLOTS / 64, VI = VSLOTS / 64;
  static_assert(KI == VI, "a row's K and V^T tiles take the same number of load instructions");
  constexpr int KVI = KI + VI;                       // 1-KB load instructions per row and tile: K0, (K1), V0, (V1)
  constexpr int SPW = KVI / QW > 0 ? KVI / QW : 1;   // of which a wave issues this many (waves beyond KVI: none)
  constexpr int TBS = QWG * 8;  // [QWG q][32 k] fp32 in 16-byte slots
  constexpr int TBI = kRQ;  // bias instructions per wave and tile
  static_assert(TBI * 64 * kWaves == TBS, "the waves share the bias slice evenly");
  constexpr int LPT = TBI + KI;

  extern __shared__ u32x4_t lds[];
  u32x4_t* tb_lds = lds;                         // [kStages][TBS]
  u32x4_t* kv_lds = lds + kStages * TBS;        // [kRows][kStages][KVS]

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int row = wave / QW, qq = wave % QW;
  const int lane = tid & 63, l32 = lane & 31, lh = lane >> 5;
  const int N = p.N, Jp = p.Jp;
  const int logical = xcd_logical_block(blockIdx.x, per_xcd);
  if (logical >= total) return;  // whole work-group leaves together
  // Order of the work-groups of one (batch element, head): blocks of kRgBlock row groups x kQcBlock query
  // ranges; inside a block the query range runs fastest, then the row group.  The work-groups resident on
  // an XCD together (about 64) are then one such block, and both streams that miss the L2 are shared: a
  // row group's K / V^T tiles by its query ranges, a query range's bias slice by the row groups.  With
  // kQcBlock query ranges or fewer (N <= 1024) this is simply: all query ranges of a row group, then the
  // next row group.
  const FlashItem item = flash_item(logical, n_qc, n_rg, kRgBlock, kQcBlock);  // of3_tiles.h
  const int bh = item.bh, qc = item.qc, rg = item.rg;
  const int i_raw = rg * kRows + row;
  const bool row_valid = i_raw < N;  // wave-uniform; idle waves still take part in the loads and barriers
  const int i = row_valid ? i_raw : N - 1;
  const int b = bh / H, h = bh % H;
  const int qwg = qc * QWG;
  const int q0 = qwg + kQW * qq;

  const size_t bih = ((size_t)b * N + i) * H + h;
  const bf16_t* Q = p.q + bih * Jp * D;
  const bf16_t* K = p.k + bih * Jp * D;
  const bf16_t* Vt = p.vt + bih * D * Jp;
  const float* tb = p.tbias + ((size_t)b * H + h) * N * Jp;
  const float* mb = p.mbias + ((size_t)b * N + i) * Jp;
  const int nkt = (N + 31) / 32;

  u32x4_t qop[kRQ][KSQ];
#pragma unroll
  for (int rq = 0; rq < kRQ; ++rq) {
    int qrow = q0 + 32 * rq + l32;
    qrow = qrow < Jp ? qrow : Jp - 1;
#pragma unroll
    for (int ks = 0; ks < KSQ; ++ks)
      qop[rq][ks] = *reinterpret_cast<const u32x4_t*>(Q + (size_t)qrow * D + 16 * ks + 8 * lh);
  }

  // bias slice: instruction n of wave w fills slots 64*(TBI*w+n)..+63; slot t holds chunk
  // (t & 7) ^ ((q >> 1) & 7) of query q = t >> 3 of the work-group's range
  uint32_t tb_off[TBI];
#pragma unroll
  for (int n = 0; n < TBI; ++n) {
    const int t = 64 * (TBI * wave + n) + lane;
    const int qloc = t >> 3, chunk = (t & 7) ^ ((qloc >> 1) & 7);
    int qrow = qwg + qloc;
    qrow = qrow < N ? qrow : N - 1;
    tb_off[n] = (uint32_t)(((size_t)qrow * Jp + 4 * chunk) * sizeof(float));
  }
  // the wave's share of its row's stage: SPW of the row's KVI load instructions, all of the K tile or all
  // of the V^T tile (the second instruction of a tile takes rows 16 further on, which flips bit 1 of
  // key4: its offset is (first ^ 32) + 1024)
  static_assert(KI == 1 || (KI == 2 && QCH == 4), "offset rule of the second instruction");
  const int slot0 = qq * SPW;               // first instruction slot of this wave
  const bool has_kv = slot0 < KVI;          // wave-uniform
  const bool is_v = slot0 >= KI;
  const int idx0 = is_v ? slot0 - KI : slot0;
  uint32_t kv_off;
  if (!is_v) {
    const int r = lane / QCH, chunk = (lane % QCH) ^ (QCH == 4 ? key4(r) : key2(r));
    kv_off = (uint32_t)((r * D + 8 * chunk) * sizeof(bf16_t));
  } else {
    const int r = lane >> 2, chunk = (lane & 3) ^ key4(r);
    kv_off = (uint32_t)((r * 32 + 8 * chunk) * sizeof(bf16_t));
  }
  if (idx0 == 1) kv_off = (kv_off ^ 32u) + 1024u;
  u32x4_t* kv_row = kv_lds + row * (kStages * KVS);
  // Loads go through buffer descriptors (scalar base, 32-bit lane offset, scalar tile offset): the
  // addresses cost one register per stream, and a load beyond its range would return zeros.
  const __amdgpu_buffer_rsrc_t tb_rsrc = buffer_rsrc(tb, (size_t)N * Jp * sizeof(float));
  const __amdgpu_buffer_rsrc_t kv_rsrc = buffer_rsrc(is_v ? Vt : K, (size_t)Jp * D * sizeof(bf16_t));
  const __amdgpu_buffer_rsrc_t mb_rsrc = buffer_rsrc(mb, (size_t)Jp * sizeof(float));
  auto issue_loads = [&](int kt, int buf) {  // buf is a constant at every call site
    u32x4_t* tdst = tb_lds + buf * TBS + 64 * TBI * wave;
    u32x4_t* kdst = kv_row + buf * KVS + (is_v ? KSLOTS : 0) + 64 * idx0;
#pragma unroll
    for (int n = 0; n < TBI; ++n)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(tb_rsrc, (void OF3_LDS_AS*)(tdst + 64 * n), 16, tb_off[n],
                                               kt * (32 * (int)sizeof(float)), 0, 0);
    const int kv_tile = kt * (32 * D * (int)sizeof(bf16_t));
    if (has_kv) {  // wave-uniform and the same in every tile: the number of loads per tile stays a constant of the wave
      __builtin_amdgcn_raw_ptr_buffer_load_lds(kv_rsrc, (void OF3_LDS_AS*)kdst, 16, kv_off, kv_tile, 0, 0);
      if (SPW == 2)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(kv_rsrc, (void OF3_LDS_AS*)(kdst + 64), 16, (kv_off ^ 32u) + 1024u,
                                                 kv_tile, 0, 0);
    }
  };
  auto load_mb = [&](int kt, uint32_t lane_off) {
    return __builtin_amdgcn_raw_buffer_load_b32(mb_rsrc, lane_off, kt * (32 * (int)sizeof(float)), 0);
  };

  const int krow = rowperm16(l32);
  const bool vvalid = krow < D;
  int k_rd[KSQ], v_rd[2];
#pragma unroll
  for (int ks = 0; ks < KSQ; ++ks) k_rd[ks] = krow * QCH + ((2 * ks + lh) ^ (QCH == 4 ? key4(krow) : key2(krow)));
#pragma unroll
  for (int s2 = 0; s2 < 2; ++s2) {
    const int vr = krow & (D - 1);
    v_rd[s2] = KSLOTS + vr * 4 + ((2 * lh + s2) ^ key4(vr));
  }
  const int tb_key = (l32 >> 1) & 7;
  const int tb_row = (kRQ * qq) * 256 + l32 * 8;

  float m_run[kRQ], l_run[kRQ], l_tot[kRQ];
  f32x16_t oacc[kRQ];
  // Head width 32, first pass: the row sums come from the matrix pipe as well.  The weights of a tile sit
  // in the B-operand registers of the P V product: lane 16 g + n holds 8 keys of query 16 (g % 2) + n.
  // Read as the B operand of a 16 x 16 x 32 product, lane 16 g + n is column n, k-group g; with an A
  // operand whose row 0 is ones over the k-groups 0 and 2 and whose row 1 is ones over the k-groups 1 and 3,
  // row 0 of the result sums query n and row 1 query 16 + n (registers 0 and 1 of lanes 0..15), over the
  // keys of both lane halves.  Two such products per tile replace sixteen additions on the vector pipe,
  // which is the busier one; the sums are those of the bf16 weights the P V product multiplies.
  f32x4_t lsum[kRQ];
  const uint32_t ones_pat = (lane == 0 || lane == 32 || lane == 17 || lane == 49) ? 0x3F803F80u : 0u;
  const u32x4_t ones_a = {ones_pat, ones_pat, ones_pat, ones_pat};

  // mask-bias k-step on the 8-deep MFMA (two registers per operand): A = [mb[key], 0, 0, 0], B = [1, 0, 0, 0],
  // both built where they are used (few tiles hold a masked or padded key)
  auto mask_step = [&](float mb_cur, f32x16_t acc) {
    const bool lo = lh == 0;  // lanes 0..31 hold k = 0..3, lanes 32..63 the unused k = 4..7
    const u32x2_t mb_op = {lo ? pack_bf16(mb_cur, 0.f) : 0u, 0u};
    const u32x2_t one_op = {lo ? 0x3F80u : 0u, 0u};
    return mfma_32x32x8(mb_op, one_op, acc);
  };
  auto offset_step = [&](float m, f32x16_t acc) {
    const bool lo = lh == 0;  // lanes 0..31 hold k = 0..3, lanes 32..63 the unused k = 4..7
    const uint32_t hi_bits = __float_as_uint(m) & 0xffff0000u;
    const float r1 = m - __uint_as_float(hi_bits);        // exact
    const uint32_t mid_bits = __float_as_uint(r1) & 0xffff0000u;
    const float r2 = r1 - __uint_as_float(mid_bits);      // exact, at most 8 significant bits
    const uint32_t sign = 0x80000000u;
    // k-slot 0: -hi, 1: -mid, 2: -lo (a bf16 is the upper half of its fp32 word)
    const u32x2_t b_op = {lo ? (((hi_bits ^ sign) >> 16) | ((mid_bits ^ sign) & 0xffff0000u)) : 0u,
                          lo ? ((__float_as_uint(r2) ^ sign) >> 16) : 0u};
    const u32x2_t a_op = {lo ? 0x3F803F80u : 0u, lo ? 0x3F80u : 0u};
    return mfma_32x32x8(a_op, b_op, acc);
  };
  // a wave of a row past the end, or whose queries all lie past the end (N not a multiple of 4 or of 64),
  // still takes part in the loads and barriers of its work-group but leaves the arithmetic out; so does
  // a 32-query tile past the end.  All of these are wave-uniform.
  const bool wave_has_work = row_valid && q0 < N;
  auto tile = [&](auto track, int buf, float mb_cur) {
    constexpr bool kTrack = decltype(track)::value;
    if (!wave_has_work) return;
    // first pass: a tile whose keys are all masked or padded adds exp2(-1.44e9 + logit) = 0 exactly to
    // every sum and is left out (a row without any unmasked key thus does nothing here, ends with the
    // row sum 0 and takes the second pass, as it has to anyway)
    if (!kTrack && __builtin_amdgcn_ballot_w64(mb_cur > kMaskedBelow) == 0) return;
    const bool has_mb = __builtin_amdgcn_ballot_w64(mb_cur != 0.f) != 0;
    const u32x4_t* tbuf = tb_lds + buf * TBS + tb_row;
    const u32x4_t* kvb = kv_row + buf * KVS;
    u32x4_t kc[KSQ], vc[2];
#pragma unroll
    for (int ks = 0; ks < KSQ; ++ks) kc[ks] = kvb[k_rd[ks]];
#pragma unroll
    for (int s2 = 0; s2 < 2; ++s2) {
      const u32x4_t v = kvb[v_rd[s2]];
      // head width 16: rows 16..31 of the operand are free; row 16 is ones (the row sum), the rest zeros
      const uint32_t fill = (krow == 16) ? 0x3F803F80u : 0u;
      const u32x4_t z = {fill, fill, fill, fill};
      vc[s2] = (D == 32 || vvalid) ? v : z;
    }
#pragma unroll
    for (int rq = 0; rq < kRQ; ++rq) {
      if (rq > 0 && q0 + 32 * rq >= N) continue;
      f32x16_t s;
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const u32x4_t t = tbuf[rq * 256 + ((4 * lh + c) ^ tb_key)];
#pragma unroll
        for (int e = 0; e < 4; ++e) s[4 * c + e] = __uint_as_float(t[e]);
      }
      if (has_mb) s = mask_step(mb_cur, s);
#pragma unroll
      for (int ks = 0; ks < KSQ; ++ks) s = mfma_32x32x16(kc[ks], qop[rq][ks], s);

      if constexpr (kTrack) {
        float mx = max3(s[0], s[1], s[2]);
#pragma unroll
        for (int v = 3; v < 15; v += 2) mx = max3(mx, s[v], s[v + 1]);
        mx = fmaxf(mx, s[15]);
        if (__builtin_amdgcn_ballot_w64(mx > m_run[rq] + kRaise) != 0) {
          // both halves of a query's lane pair take the same new offset; an offset of moderate size is
          // replaced by 0 (any offset gives the same softmax, and 0 needs no subtraction below)
          float m_new = fmaxf(m_run[rq], fmaxf(mx, xhalf(mx)));
          m_new = __builtin_fabsf(m_new) <= kSnap ? 0.f : m_new;
          const float alpha = fast_exp2(m_run[rq] - m_new);  // exp2(-inf) = 0 on the first tile
          l_run[rq] *= alpha;
#pragma unroll
          for (int v = 0; v < 16; ++v) oacc[rq][v] *= alpha;
          m_run[rq] = m_new;
        }
        // A query whose offset is not 0 (logits beyond +-32, or only masked keys so far) gets it
        // subtracted by one more k-step, A = [1, 1, 1, 0 ...], B = -[hi, mid, lo, 0 ...] with the fp32
        // offset split exactly into three bf16 terms: s - m without rounding, after (tb + mb) + q.k has
        // been formed, so a row of masked keys still ends with equal logits.  Rare; the usual tile goes
        // straight to the exponentials.
        if (__builtin_amdgcn_ballot_w64(m_run[rq] != 0.f) != 0) s = offset_step(m_run[rq], s);
      }
      // softmax weights: fp32 row sum (the reference normalises with the fp32 sum and rounds the
      // weights to bf16 afterwards, attention.py:130-133), bf16 weights for the P V product
      float rs = l_run[rq];
      u32x4_t pop0, pop1;
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        const float e0 = fast_exp2(s[2 * w]), e1 = fast_exp2(s[2 * w + 1]);
        if (D == 32 && kTrack) {
          rs += e0;
          rs += e1;
        }
        pop0[w] = pack_bf16(e0, e1);
      }
      oacc[rq] = mfma_32x32x16(vc[0], pop0, oacc[rq]);
      if (D == 32 && !kTrack) lsum[rq] = mfma_16x16x32(ones_a, pop0, lsum[rq]);
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        const float e0 = fast_exp2(s[8 + 2 * w]), e1 = fast_exp2(s[8 + 2 * w + 1]);
        if (D == 32 && kTrack) {
          rs += e0;
          rs += e1;
        }
        pop1[w] = pack_bf16(e0, e1);
      }
      oacc[rq] = mfma_32x32x16(vc[1], pop1, oacc[rq]);
      if (D == 32 && !kTrack) lsum[rq] = mfma_16x16x32(ones_a, pop1, lsum[rq]);
      l_run[rq] = rs;
    }
  };

  const uint32_t mb_off = krow * sizeof(float);
  auto pass = [&](auto track) {
#pragma unroll
    for (int rq = 0; rq < kRQ; ++rq) {
      m_run[rq] = decltype(track)::value ? -__builtin_inff() : 0.f;
      l_run[rq] = 0.f;
      oacc[rq] = zero16();
      lsum[rq] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    }
    float mb_next = __uint_as_float(load_mb(0, mb_off));
    issue_loads(0, 0);
    auto step = [&](int kt, int buf) {  // buf is a constant at both call sites: LDS addresses are immediates
      wait_vmcnt<0>();               // this wave's loads of tile kt (and its mask-bias values) have landed ...
      __builtin_amdgcn_s_barrier();  // ... and everybody's; nobody reads tile kt-1's buffers any more
      compiler_fence();
      const float mb_cur = mb_next;
      const int ktn = kt + 1 < nkt ? kt + 1 : nkt - 1;
      mb_next = __uint_as_float(load_mb(ktn, mb_off));
      issue_loads(ktn, buf ^ 1);
      tile(track, buf, mb_cur);
      compiler_fence();
    };
    for (int kt = 0; kt < nkt; kt += 2) {
      step(kt, 0);
      if (kt + 1 < nkt) step(kt + 1, 1);
    }
    wait_vmcnt<0>();  // the loads issued past the end must not outlive the pass (or the work-group's LDS)
#pragma unroll
    for (int rq = 0; rq < kRQ; ++rq) {
      if (D == 32 && decltype(track)::value) {
        l_tot[rq] = l_run[rq] + xhalf(l_run[rq]);
      } else if (D == 32) {
        const float lo = __shfl(lsum[rq][0], l32 & 15, 64), hi = __shfl(lsum[rq][1], l32 & 15, 64);
        l_tot[rq] = (l32 & 16) ? hi : lo;
      } else {
        // V^T row 16 (ones) is result row 16: register 0 of the upper lane half, same query column
        const float mine = oacc[rq][0], other = xhalf(mine);
        l_tot[rq] = lh ? mine : other;
      }
    }
  };

  // First pass: offset 0 for every query, no running maximum.  It is exact whenever a query's
  // logits stay in a range where exp2 neither overflows nor loses its largest terms, which the
  // row sum itself tells: 2^-60 <= sum <= 2^60 (an overflow leaves +inf in the sum, a row of masked
  // keys leaves 0).  If any query of the work-group fails that test, the whole work-group (its
  // loads and barriers are collective) runs the pass again with running maxima.
  pass(std::false_type{});
  {
    bool bad = false;
#pragma unroll
    for (int rq = 0; rq < kRQ; ++rq) {
      const bool in_range = l_tot[rq] >= 0x1p-60f && l_tot[rq] <= 0x1p60f;  // false for NaN too
      bad |= row_valid && (q0 + 32 * rq + l32 < N) && !in_range;
    }
    if (__syncthreads_or(bad)) pass(std::true_type{});
  }

  if (row_valid && 16 * lh < D) {
#pragma unroll
    for (int rq = 0; rq < kRQ; ++rq) {
      const int qrow = q0 + 32 * rq + l32;
      if (qrow >= N) continue;
      const float inv = fast_rcp(l_tot[rq]);
      u32x4_t o0, o1;
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        o0[w] = pack_bf16(oacc[rq][2 * w] * inv, oacc[rq][2 * w + 1] * inv);
        o1[w] = pack_bf16(oacc[rq][8 + 2 * w] * inv, oacc[rq][8 + 2 * w + 1] * inv);
      }
      bf16_t* dst = p.o + (((size_t)b * N + i) * N + qrow) * HD + h * D + 16 * lh;
      *reinterpret_cast<u32x4_t*>(dst) = o0;
      *reinterpret_cast<u32x4_t*>(dst + 8) = o1;
    }
  }
}


template <int D, int QW>
constexpr int lds_bytes() {
  return (kStages * kQW * QW * 8 + kRows * kStages * (32 * (D / 8) + D * 4)) * 16;
}

template <int D, int QW>
hipError_t launch(const TriattnFlashArgs& a, hipStream_t stream) {
  static int cache[kMaxDevices];
  int configured = 0;
  hipError_t e = per_device(
      cache,
      [&](int, int* v) {
        *v = 1;
        return hipFuncSetAttribute(reinterpret_cast<const void*>(&triattn_flash_kernel<D, QW>),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, (lds_bytes<D, QW>()));
      },
      &configured);
  if (e != hipSuccess) return e;
  const int n_qc = (a.N + kQW * QW - 1) / (kQW * QW), n_rg = (a.N + kRows - 1) / kRows;
  const long total = (long)n_qc * n_rg * a.B * a.H;
  const int per_xcd = (int)((total + 7) / 8);
  constexpr int kLds = lds_bytes<D, QW>();
  triattn_flash_kernel<D, QW><<<dim3(per_xcd * 8), dim3(64 * kRows * QW), kLds, stream>>>(a, n_qc, n_rg, (int)total,
                                                                                          per_xcd);
  return hipGetLastError();
}

}  // namespace

hipError_t triattn_flash_launch(const TriattnFlashArgs& args, int D, hipStream_t stream) {
  if (args.H != 4) return hipErrorInvalidValue;
  const bool wide = args.N >= OF3_FLASH_WIDE_FROM;
  if (D == 32) return wide ? launch<32, 4>(args, stream) : launch<32, 2>(args, stream);
  if (D == 16) return wide ? launch<16, 4>(args, stream) : launch<16, 2>(args, stream);
  return hipErrorInvalidValue;
}

}  // namespace of3

// Triangle-attention core (attention.py:94-135 with the two biases of tri_att.py:134-140):
//     s[q][k] = q.k + mb[i][k] + tb[h][q][k];  p = softmax_k(s);  o[q] = sum_k p[q][k] v[k]
// for every (batch, row i, head h), flash style: 32-key tiles, running maximum and sum in
// fp32, no [N][N] logits in memory.  Inputs come from the projection pass already
// multiplied by log2(e) (q also by 1/sqrt(D)), so exp() is the hardware exp2.
//
// With head width 16 or 32 the kernel is bound by the softmax's vector work and by
// latencies, not by the MFMAs, so the organisation keeps the vector pipe fed:
//  * work-group = 8 waves = 8 consecutive rows i of one (head, 128-query range).  The
//    triangle bias of that range does not depend on i: each 32-key slice of it is brought
//    into LDS once per work-group and every wave reads it straight into the MFMA
//    accumulator, which adds it for free.
//  * everything a key tile needs (the work-group's bias slice, the wave's own K tile and
//    V^T tile) travels global -> LDS with direct-to-LDS loads, one tile ahead, into
//    double buffers; the only wait is one vmcnt(0) + barrier per key tile, a whole tile of
//    arithmetic after the loads were issued.  The XOR swizzles are applied on the global
//    side (a lane picks which 16-byte chunk it fetches for its fixed LDS slot).
//  * S^T = K Q^T: A = K tile (row r of the tile is key rowperm16(r), so a lane ends up with
//    16 consecutive keys of one query), B = Q tile (registers).  O^T = V^T P^T: A = V^T,
//    B = P^T taken directly from the S^T accumulator registers (no cross-lane movement).
//  * inside a key tile the four 32-query tiles are software pipelined: the bias reads and
//    the q.k MFMAs of the next query tile are issued in the middle of the current one's
//    exponentials, so a wave overlaps its own matrix and vector work.
//  * the running maximum is only raised when a logit exceeds it by more than 2^8 (checked
//    wave-wide with one ballot); otherwise a logit costs one subtract, one exp2, one add
//    and half a pack.  Any common offset gives the same softmax; the bound keeps every
//    term far from overflow.
//  * the mask bias of a key tile rides on one more k-step of the S^T product (A = [mb[key],
//    0, ...], B = [1, 0, ...]) right after the triangle bias, i.e. (tb + mb) + q.k in the
//    fp32 accumulator: masked keys get weight exactly 0, padded keys (N not a multiple of
//    32) carry -inf, and a fully masked row degenerates to a uniform average over all real
//    keys exactly as the reference's does (-1e9 absorbs the logits in fp32).  A key tile whose
//    32 mask biases are all zero (checked wave-wide once per tile) skips that k-step.
#include "of3_device.h"
#include "of3_kernels.h"
#include "of3_launch.h"

namespace of3 {

namespace {

#define OF3_GLOBAL_AS __attribute__((address_space(1)))
#define OF3_LDS_AS __attribute__((address_space(3)))

constexpr int kRows = 8;          // rows i (= waves) per work-group
constexpr int kRQ = 4;            // 32-query tiles per wave
constexpr float kRaise = 8.0f;    // raise the running maximum only beyond 2^8
constexpr int kTbSlots = kRQ * 32 * 8;  // 16-byte slots of one [32*kRQ q][32 k] fp32 bias slice
constexpr int kTbLoads = kRQ * 4 / kRows;  // direct-to-LDS instructions (8 queries each) per wave and slice
static_assert(kTbLoads * kRows == kRQ * 4, "the bias slice is split evenly over the waves");
constexpr int kStages = 3;        // LDS ring: tiles kt (in use), kt+1 (landing or landed), kt+2 (requested)

__device__ __forceinline__ float xhalf(float v) { return __shfl_xor(v, 32, 64); }
__device__ __forceinline__ void compiler_fence() { __asm__ volatile("" ::: "memory"); }
template <int N>
__device__ __forceinline__ void wait_vmcnt() {  // vmcnt(N) only (gfx9 encoding, N < 16)
  static_assert(N >= 0 && N < 16, "low field only");
  __builtin_amdgcn_s_waitcnt(0x0F70 | N);
}

// swizzle keys of the K / V^T tiles in LDS: rows are read in the order rowperm16(lane), i.e.
// {x..x+3, x+16..x+19, x+4..x+7, x+20..x+23} per 16 lanes; (row & 1, key) must differ inside
// every group of 8 lanes and (row & 3, key) inside every group of 16
__device__ __forceinline__ int key4(int row) {  // 4 chunks (64 bytes) per row
  return ((((row >> 4) ^ (row >> 1)) & 1) << 1) | (((row >> 2) ^ (row >> 1)) & 1);
}
__device__ __forceinline__ int key2(int row) { return (row >> 4) & 1; }  // 2 chunks per row

template <int D>
__global__ __launch_bounds__(64 * kRows) void triattn_flash_kernel(TriattnFlashArgs p, int n_qc, int n_rg, int total,
                                                                   int per_xcd) {
  constexpr int H = 4;
  constexpr int HD = H * D;
  constexpr int KSQ = D / 16;            // k-steps of the q.k product
  constexpr int QCH = D / 8;             // 16-byte chunks per K row
  constexpr int KSLOTS = 32 * QCH;       // K tile: 32 keys x D
  constexpr int VSLOTS = D * 4;          // V^T tile: D channels x 32 keys
  constexpr int KVS = KSLOTS + VSLOTS;   // one wave's stage
  constexpr int KI = KSLOTS / 64, VI = VSLOTS / 64;  // direct-to-LDS instructions per tile

  extern __shared__ u32x4_t lds[];
  u32x4_t* tb_lds = lds;                           // [kStages][kTbSlots]
  u32x4_t* kv_lds = lds + kStages * kTbSlots;      // [kRows][kStages][KVS]

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63, l32 = lane & 31, lh = lane >> 5;
  const int N = p.N, Jp = p.Jp;
  // Work-groups that differ only in the query range read the same K and V rows: they get
  // consecutive logical ids, which the XCD-aware numbering keeps on one XCD (one L2).
  const int logical = xcd_logical_block(blockIdx.x, per_xcd);
  if (logical >= total) return;  // whole work-group leaves together
  const int qc = logical % n_qc;
  const int rg = (logical / n_qc) % n_rg;
  const int bh = logical / (n_qc * n_rg);
  const int i_raw = rg * kRows + wave;
  const bool row_valid = i_raw < N;          // wave-uniform; idle waves still take part in the loads and barriers
  const int i = row_valid ? i_raw : N - 1;
  const int b = bh / H, h = bh % H;
  const int q0 = qc * (32 * kRQ);

  const size_t bih = ((size_t)b * N + i) * H + h;
  const bf16_t* Q = p.q + bih * Jp * D;
  const bf16_t* K = p.k + bih * Jp * D;
  const bf16_t* Vt = p.vt + bih * D * Jp;
  const float* tb = p.tbias + ((size_t)b * H + h) * N * Jp;
  const float* mb = p.mbias + ((size_t)b * N + i) * Jp;
  const int nkt = (N + 31) / 32;

  // ---- query operands (B side of S^T = K Q^T) stay in registers
  u32x4_t qop[kRQ][KSQ];
#pragma unroll
  for (int rq = 0; rq < kRQ; ++rq) {
    int qrow = q0 + 32 * rq + l32;
    qrow = qrow < Jp ? qrow : Jp - 1;
#pragma unroll
    for (int ks = 0; ks < KSQ; ++ks)
      qop[rq][ks] = *reinterpret_cast<const u32x4_t*>(Q + (size_t)qrow * D + 16 * ks + 8 * lh);
  }

  // ---- direct-to-LDS sources.  LDS slot of an instruction = its base + lane.
  // bias slice: instruction n of wave w fills slots 64*(2w+n)..+63; slot t holds chunk
  // (t & 7) ^ ((q >> 1) & 7) of query q = t >> 3 (128-byte rows of 32 keys)
  // (byte offsets from wave-uniform bases, so that the loads use scalar base + 32-bit lane offset)
  uint32_t tb_off[kTbLoads];
#pragma unroll
  for (int n = 0; n < kTbLoads; ++n) {
    const int t = 64 * (kTbLoads * wave + n) + lane;
    const int qloc = t >> 3, chunk = (t & 7) ^ ((qloc >> 1) & 7);
    int qrow = q0 + qloc;
    qrow = qrow < N ? qrow : N - 1;
    tb_off[n] = (uint32_t)(((size_t)qrow * Jp + 4 * chunk) * sizeof(float));
  }
  // K tile: slot t holds chunk (t % QCH) ^ key(row) of key row t / QCH
  uint32_t k_off[KI];
#pragma unroll
  for (int n = 0; n < KI; ++n) {
    const int t = 64 * n + lane;
    const int row = t / QCH, chunk = (t % QCH) ^ (QCH == 4 ? key4(row) : key2(row));
    k_off[n] = (uint32_t)((row * D + 8 * chunk) * sizeof(bf16_t));
  }
  // V^T tile: slot t holds chunk (t & 3) ^ key4(row) of channel row t >> 2 (64-byte rows of 32 keys)
  uint32_t v_off[VI];
#pragma unroll
  for (int n = 0; n < VI; ++n) {
    const int t = 64 * n + lane;
    const int row = t >> 2, chunk = (t & 3) ^ key4(row);
    v_off[n] = (uint32_t)((row * 32 + 8 * chunk) * sizeof(bf16_t));
  }
  u32x4_t* kv_mine = kv_lds + wave * (kStages * KVS);
  auto issue_loads = [&](int kt, int buf) {
    u32x4_t* tdst = tb_lds + buf * kTbSlots + 64 * kTbLoads * wave;
    u32x4_t* kdst = kv_mine + buf * KVS;
    const char* tbase = reinterpret_cast<const char*>(tb + 32 * kt);
    const char* kbase = reinterpret_cast<const char*>(K + (size_t)kt * (32 * D));
    const char* vbase = reinterpret_cast<const char*>(Vt + (size_t)kt * (32 * D));
#pragma unroll
    for (int n = 0; n < kTbLoads; ++n)
      __builtin_amdgcn_global_load_lds((const void OF3_GLOBAL_AS*)(tbase + tb_off[n]),
                                       (void OF3_LDS_AS*)(tdst + 64 * n), 16, 0, 0);
#pragma unroll
    for (int n = 0; n < KI; ++n)
      __builtin_amdgcn_global_load_lds((const void OF3_GLOBAL_AS*)(kbase + k_off[n]),
                                       (void OF3_LDS_AS*)(kdst + 64 * n), 16, 0, 0);
#pragma unroll
    for (int n = 0; n < VI; ++n)
      __builtin_amdgcn_global_load_lds((const void OF3_GLOBAL_AS*)(vbase + v_off[n]),
                                       (void OF3_LDS_AS*)(kdst + KSLOTS + 64 * n), 16, 0, 0);
  };

  // ---- operand read slots
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
  // bias slot this lane reads for tile rq, chunk c: rq*256 + l32*8 + ((4*lh + c) ^ key), key =
  // (l32 >> 1) & 7: the 16 lanes of one read phase hold 16 consecutive queries, two 128-byte
  // rows per 256-byte bank window, so queries of equal parity need distinct keys
  int tb_rd[4];
#pragma unroll
  for (int c = 0; c < 4; ++c) tb_rd[c] = l32 * 8 + ((4 * lh + c) ^ ((l32 >> 1) & 7));

  float m_run[kRQ], l_run[kRQ];
  f32x16_t oacc[kRQ];
#pragma unroll
  for (int rq = 0; rq < kRQ; ++rq) {
    m_run[rq] = -__builtin_inff();
    l_run[rq] = 0.f;
    oacc[rq] = zero16();
  }

  // One key tile.
  // Mask bias of a tile: one more k-step of the S^T product with A = [mb[key], 0, ...] and
  // B = [1, 0, ...] adds mb[key] to every query's logit inside the matrix pipe, right after
  // the triangle bias ((tb + mb) + q.k).  bf16 holds 0 and -inf exactly and -1e9*log2(e) to
  // 3 digits, which is all a mask bias has to be.
  float mb_cur = 0.f;  // mb[32*kt + rowperm16(l32)] of the current tile
  const u32x4_t one_op = {lh == 0 ? 0x3F80u : 0u, 0u, 0u, 0u};
  auto tile = [&](int buf) {
    const u32x4_t mb_op = {lh == 0 ? pack_bf16(mb_cur, 0.f) : 0u, 0u, 0u, 0u};
    // a tile without a masked or padded key (the usual case) adds nothing: its mask k-step is skipped
    const bool has_mb = __builtin_amdgcn_ballot_w64(mb_cur != 0.f) != 0;
    const u32x4_t* tbuf = tb_lds + buf * kTbSlots;
    const u32x4_t* kvb = kv_mine + buf * KVS;
    u32x4_t kc[KSQ], vc[2];
#pragma unroll
    for (int ks = 0; ks < KSQ; ++ks) kc[ks] = kvb[k_rd[ks]];
#pragma unroll
    for (int s2 = 0; s2 < 2; ++s2) {
      const u32x4_t v = kvb[v_rd[s2]];
      const u32x4_t z = {0u, 0u, 0u, 0u};
      vc[s2] = vvalid ? v : z;
    }
    auto bias_init = [&](int rq) {
      f32x16_t s;
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const u32x4_t t = tbuf[rq * 256 + tb_rd[c]];
#pragma unroll
        for (int e = 0; e < 4; ++e) s[4 * c + e] = __uint_as_float(t[e]);
      }
      return s;
    };

    f32x16_t s = bias_init(0);
    if (has_mb) s = mfma_32x32x16(mb_op, one_op, s);
#pragma unroll
    for (int ks = 0; ks < KSQ; ++ks) s = mfma_32x32x16(kc[ks], qop[0][ks], s);

#pragma unroll
    for (int rq = 0; rq < kRQ; ++rq) {
      // bias of the next query tile: LDS reads in flight during the maximum search
      f32x16_t sn;
      if (rq + 1 < kRQ) sn = bias_init(rq + 1);

      float mx = fmaxf(s[0], s[1]);
#pragma unroll
      for (int v = 2; v < 16; v += 2) mx = fmaxf(fmaxf(mx, s[v]), s[v + 1]);
      if (__builtin_amdgcn_ballot_w64(mx > m_run[rq] + kRaise) != 0) {
        // both halves of a query's lane pair take the same new maximum
        const float m_new = fmaxf(m_run[rq], fmaxf(mx, xhalf(mx)));
        const float alpha = fast_exp2(m_run[rq] - m_new);  // exp2(-inf) = 0 on the first tile
        l_run[rq] *= alpha;
#pragma unroll
        for (int v = 0; v < 16; ++v) oacc[rq][v] *= alpha;
        m_run[rq] = m_new;
      }
      const float m = m_run[rq];

      // exponentials in groups; the next tile's q.k MFMAs and this tile's P V MFMAs are
      // slipped in between so that the matrix pipe works under the vector work.  The row
      // sum is taken over the bf16-rounded weights (the ones the P V product uses), two per
      // instruction with the bf16 dot product.
      float rs = l_run[rq];  // this lane's 16 keys; the two halves are combined at the end
      auto expw = [&](int w) {  // weights 2w, 2w+1 -> one packed register
        const uint32_t pk = pack_bf16(fast_exp2(s[2 * w] - m), fast_exp2(s[2 * w + 1] - m));
        rs = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, pk), __builtin_bit_cast(bf16x2_t, 0x3F803F80u),
                                             rs, false);
        return pk;
      };
      u32x4_t pop0, pop1;
#pragma unroll
      for (int w = 0; w < 4; ++w) pop0[w] = expw(w);
      __builtin_amdgcn_sched_barrier(0);
      if (rq + 1 < kRQ) {
        if (has_mb) sn = mfma_32x32x16(mb_op, one_op, sn);
        sn = mfma_32x32x16(kc[0], qop[rq + 1 < kRQ ? rq + 1 : 0][0], sn);
      }
      __builtin_amdgcn_sched_barrier(0);
      pop1[0] = expw(4);
      pop1[1] = expw(5);
      __builtin_amdgcn_sched_barrier(0);
      if (KSQ == 2 && rq + 1 < kRQ) sn = mfma_32x32x16(kc[KSQ - 1], qop[rq + 1 < kRQ ? rq + 1 : 0][KSQ - 1], sn);
      oacc[rq] = mfma_32x32x16(vc[0], pop0, oacc[rq]);
      __builtin_amdgcn_sched_barrier(0);
      pop1[2] = expw(6);
      pop1[3] = expw(7);
      __builtin_amdgcn_sched_barrier(0);
      oacc[rq] = mfma_32x32x16(vc[1], pop1, oacc[rq]);
      __builtin_amdgcn_sched_barrier(0);
      l_run[rq] = rs;
      if (rq + 1 < kRQ) s = sn;
    }
  };

  constexpr int LPT = kTbLoads + KI + VI;  // direct-to-LDS instructions per tile and wave
  float mb_next = mb[krow];
  constexpr int PD = kStages - 1;  // prefetch distance in tiles
#pragma unroll
  for (int t = 0; t < PD; ++t)
    if (t < nkt) issue_loads(t, t);
  int buf = 0;  // kt % kStages
  for (int kt = 0; kt < nkt; ++kt) {
    // this wave's loads of tile kt have landed (those of later tiles may still be in flight) ...
    if (PD >= 2 && kt + PD - 1 < nkt) wait_vmcnt<(PD - 1) * LPT>();
    else wait_vmcnt<0>();
    __builtin_amdgcn_s_barrier();      // ... and everybody's; nobody reads tile kt-1's buffers any more
    compiler_fence();
    mb_cur = mb_next;
    if (kt + 1 < nkt) mb_next = mb[32 * (kt + 1) + krow];  // an ordinary load, issued before the prefetch
    if (kt + PD < nkt) issue_loads(kt + PD, buf == 0 ? kStages - 1 : buf - 1);
    tile(buf);
    buf = buf == kStages - 1 ? 0 : buf + 1;
    compiler_fence();
  }

  // ---- finalize: lane (query l32, half lh) owns head channels 16*lh + v
  float l_tot[kRQ];
#pragma unroll
  for (int rq = 0; rq < kRQ; ++rq) l_tot[rq] = l_run[rq] + xhalf(l_run[rq]);  // all lanes take part
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

template <int D>
constexpr int lds_bytes() {
  return (kStages * kTbSlots + kRows * kStages * (32 * (D / 8) + D * 4)) * 16;
}

template <int D>
hipError_t launch(const TriattnFlashArgs& a, hipStream_t stream) {
  auto kern = triattn_flash_kernel<D>;
  static int cache[kMaxDevices];
  int configured = 0;
  hipError_t e = per_device(
      cache,
      [&](int, int* v) {
        *v = 1;
        return hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                   lds_bytes<D>());
      },
      &configured);
  if (e != hipSuccess) return e;
  const int n_qc = (a.N + 32 * kRQ - 1) / (32 * kRQ), n_rg = (a.N + kRows - 1) / kRows;
  const long total = (long)n_qc * n_rg * a.B * a.H;
  const int per_xcd = (int)((total + 7) / 8);
  hipLaunchKernelGGL(kern, dim3(per_xcd * 8), dim3(64 * kRows), lds_bytes<D>(), stream, a, n_qc, n_rg, (int)total,
                     per_xcd);
  return hipGetLastError();
}

}  // namespace

hipError_t triattn_flash_launch(const TriattnFlashArgs& args, int D, hipStream_t stream) {
  if (args.H != 4) return hipErrorInvalidValue;
  if (D == 32) return launch<32>(args, stream);
  if (D == 16) return launch<16>(args, stream);
  return hipErrorInvalidValue;
}

}  // namespace of3

// Triangle-attention core (attention.py:94-135 with the two biases of tri_att.py:134-140):
//     s[q][k] = q.k + mb[i][k] + tb[h][q][k];  p = softmax_k(s);  o[q] = sum_k p[q][k] v[k]
// for every (batch, row i, head h), flash style: 32-key tiles, running maximum and sum in
// fp32, no [N][N] logits in memory.  Inputs come from the projection pass already
// multiplied by log2(e) (q also by 1/sqrt(D)), so exp() is the hardware exp2.
//
// With head width 16 or 32 the kernel is bound by the softmax's VALU work, not by the
// MFMAs, so the organisation minimises vector instructions per logit:
//  * work-group = 8 waves = 8 consecutive rows i of one (head, 128-query range).  The
//    triangle bias of that range does not depend on i: each 32-key slice of it is brought
//    into LDS once per work-group (double-buffered) and every wave reads it
//    straight into the MFMA accumulator, which adds it for free.
//  * S^T = K Q^T: A = K tile (row r of the tile is key rowperm16(r), so a lane ends up with
//    16 consecutive keys of one query), B = Q tile.  O^T = V^T P^T: A = V^T, B = P^T taken
//    directly from the S^T accumulator registers (no cross-lane movement).  K and V^T are
//    loaded straight from global memory in operand layout and prefetched one tile ahead.
//  * the running maximum is only raised when a logit exceeds it by more than 2^8 (checked
//    wave-wide with one ballot); otherwise the tile costs per logit one subtract, one exp2,
//    one add and half a pack.  Any common offset gives the same softmax; the bound keeps
//    every term far from overflow.
//  * rows without masked keys never touch the mask bias.  Otherwise, and in the last tile
//    when N is not a multiple of 32 (padded keys carry -inf), it is added to the triangle
//    bias first: masked keys get weight exactly 0, and a fully masked row degenerates to a
//    uniform average over all real keys exactly as the reference's does (-1e9 absorbs the
//    logits in fp32).
#include "of3_device.h"
#include "of3_kernels.h"

namespace of3 {

namespace {

constexpr int kRows = 8;          // rows i (= waves) per work-group
constexpr int kRQ = 4;            // 32-query tiles per wave
constexpr float kRaise = 8.0f;    // raise the running maximum only beyond 2^8

__device__ __forceinline__ float xhalf(float v) { return __shfl_xor(v, 32, 64); }

template <int D>
__global__ __launch_bounds__(64 * kRows) void triattn_flash_kernel(TriattnFlashArgs p, int n_qc, int n_rg, int total,
                                                                   int per_xcd) {
  constexpr int H = 4;
  constexpr int HD = H * D;
  constexpr int KSQ = D / 16;           // k-steps of the q.k product
  constexpr int TBQ = 32 * 8;           // u32x4 slots of one 32 x 32 fp32 bias tile
  constexpr int TBBUF = kRQ * TBQ;      // one key slice of the whole query range

  constexpr int QCH = D / 8;             // 16-byte chunks per query row
  constexpr int QSLOTS = 32 * kRQ * QCH; // one wave's 128 query rows
  __shared__ u32x4_t tb_lds[2 * TBBUF];          // 32 KB
  __shared__ u32x4_t q_lds[kRows * QSLOTS];      // 64 KB (D = 32): every wave's own query operands

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
  const bool row_valid = i_raw < N;          // wave-uniform; idle waves still take part in the barriers
  const int i = row_valid ? i_raw : N - 1;
  const int b = bh / H, h = bh % H;
  const int q0 = qc * (32 * kRQ);

  const size_t bih = ((size_t)b * N + i) * H + h;
  const bf16_t* Q = p.q + bih * Jp * D;
  const bf16_t* K = p.k + bih * Jp * D;
  const bf16_t* Vt = p.vt + bih * D * Jp;
  const float* tb = p.tbias + ((size_t)b * H + h) * N * Jp;
  const float* mb = p.mbias + ((size_t)b * N + i) * Jp;

  // ---- does this row have masked keys at all?  (wave-uniform)
  bool row_masked = false;
  {
    float acc = 0.f;
    for (int j = lane * 4; j < N; j += 256) {
      const float4 t4 = *reinterpret_cast<const float4*>(mb + j);  // j+3 < Jp; entries >= N are -inf
      acc += (j < N ? t4.x : 0.f) + (j + 1 < N ? t4.y : 0.f) + (j + 2 < N ? t4.z : 0.f) + (j + 3 < N ? t4.w : 0.f);
    }
    row_masked = __builtin_amdgcn_ballot_w64(acc != 0.f) != 0;
  }
  const bool tail_keys = (N & 31) != 0;
  const int nkt = (N + 31) / 32;

  // ---- query operands (B side of S^T = K Q^T): parked in LDS, 128 rows per wave, chunk
  // index XOR-ed with a row key so that the operand reads (8 lanes = 8 consecutive rows, same
  // chunk) are conflict free; fetched again for every key tile instead of living in 32 VGPRs
  u32x4_t* q_mine = q_lds + wave * QSLOTS;
  auto q_key = [](int r) { return D == 32 ? ((r >> 1) & 3) : ((r >> 2) & 1); };
  {
    constexpr int RPI = 64 / QCH;  // query rows per wave instruction
#pragma unroll
    for (int it = 0; it < 32 * kRQ / RPI; ++it) {
      const int r = it * RPI + lane / QCH, c = lane % QCH;
      int qrow = q0 + r;
      qrow = qrow < Jp ? qrow : Jp - 1;
      q_mine[r * QCH + (c ^ q_key(r))] = *reinterpret_cast<const u32x4_t*>(Q + (size_t)qrow * D + 8 * c);
    }
  }
  int q_rd[KSQ];
#pragma unroll
  for (int ks = 0; ks < KSQ; ++ks) q_rd[ks] = l32 * QCH + ((2 * ks + lh) ^ q_key(l32));

  // ---- triangle-bias slices: 128 queries x 32 keys fp32 = 16 KB per key tile, fetched by
  // the whole work-group (two 16-byte pieces per thread, 8 lanes per 128-byte query row),
  // held in registers during the current tile's arithmetic and written to the other LDS
  // buffer afterwards.  LDS slot of (tile rq, query r, chunk c) = rq*256 + r*8 + (c ^ (r & 7)).
  const float* tb_src[2];
  int tb_dst[2];
#pragma unroll
  for (int n = 0; n < 2; ++n) {
    const int qloc = 64 * n + (tid >> 3), chunk = tid & 7;  // query within the 128 range
    int qrow = q0 + qloc;
    qrow = qrow < N ? qrow : N - 1;
    tb_src[n] = tb + (size_t)qrow * Jp + 4 * chunk;
    tb_dst[n] = (qloc >> 5) * TBQ + (qloc & 31) * 8 + (chunk ^ (qloc & 7));
  }
  auto load_tb = [&](int kt, u32x4_t (&r)[2]) {
#pragma unroll
    for (int n = 0; n < 2; ++n) r[n] = *reinterpret_cast<const u32x4_t*>(tb_src[n] + 32 * kt);
  };
  auto store_tb = [&](const u32x4_t (&r)[2], int buf) {
#pragma unroll
    for (int n = 0; n < 2; ++n) tb_lds[buf * TBBUF + tb_dst[n]] = r[n];
  };

  // ---- key / value operands of one tile, loaded in operand layout
  const int krow = rowperm16(l32);
  const bool vvalid = krow < D;
  auto load_kv = [&](int kt, u32x4_t (&kop)[KSQ], u32x4_t (&vop)[2]) {
    const int key0 = 32 * kt;
#pragma unroll
    for (int s = 0; s < KSQ; ++s)
      kop[s] = *reinterpret_cast<const u32x4_t*>(K + (size_t)(key0 + krow) * D + 16 * s + 8 * lh);
#pragma unroll
    for (int s2 = 0; s2 < 2; ++s2) {
      u32x4_t v = {0u, 0u, 0u, 0u};
      if (vvalid) v = *reinterpret_cast<const u32x4_t*>(Vt + (size_t)kt * (D * 32) + krow * 32 + 16 * lh + 8 * s2);
      vop[s2] = v;
    }
  };

  float m_run[kRQ], l_run[kRQ];
  f32x16_t oacc[kRQ];
#pragma unroll
  for (int rq = 0; rq < kRQ; ++rq) {
    m_run[rq] = -__builtin_inff();
    l_run[rq] = 0.f;
    oacc[rq] = zero16();
  }

  u32x4_t kop[2][KSQ], vop[2][2], tbr[2];
  load_tb(0, tbr);
  load_kv(0, kop[0], vop[0]);
  store_tb(tbr, 0);

  // the bias slot this lane reads for tile rq, chunk c: rq*256 + l32*8 + ((4*lh + c) ^ (l32 & 7))
  const int tb_rd = l32 * 8;
  const int tb_key = l32 & 7;

  auto tile = [&](int kt, const u32x4_t (&kc)[KSQ], const u32x4_t (&vc)[2], const u32x4_t* tbuf) {
    const bool use_mb = row_masked || (tail_keys && kt == nkt - 1);  // wave-uniform
    const float* mbt = mb + 32 * kt + 16 * lh;
#pragma unroll
    for (int rq = 0; rq < kRQ; ++rq) {
      f32x16_t s;
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const u32x4_t t = tbuf[rq * TBQ + tb_rd + ((4 * lh + c) ^ tb_key)];
#pragma unroll
        for (int e = 0; e < 4; ++e) s[4 * c + e] = __uint_as_float(t[e]);
      }
      if (use_mb) {
#pragma unroll
        for (int c4 = 0; c4 < 4; ++c4) {
          const float4 t4 = *reinterpret_cast<const float4*>(mbt + 4 * c4);  // same 64 bytes for every rq: L1 hits
          s[4 * c4] += t4.x;
          s[4 * c4 + 1] += t4.y;
          s[4 * c4 + 2] += t4.z;
          s[4 * c4 + 3] += t4.w;
        }
      }
#pragma unroll
      for (int ks = 0; ks < KSQ; ++ks) s = mfma_32x32x16(kc[ks], q_mine[rq * 32 * QCH + q_rd[ks]], s);

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
      float rs = 0.f;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        s[v] = fast_exp2(s[v] - m);
        rs += s[v];
      }
      l_run[rq] += rs;  // this lane's 16 keys; the two halves are combined at the end
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2) {
        u32x4_t pop;
#pragma unroll
        for (int w = 0; w < 4; ++w) pop[w] = pack_bf16(s[8 * s2 + 2 * w], s[8 * s2 + 2 * w + 1]);
        oacc[rq] = mfma_32x32x16(vc[s2], pop, oacc[rq]);
      }
      __builtin_amdgcn_sched_barrier(0);  // one query tile at a time keeps the live registers within budget
    }
  };

  for (int kt = 0; kt < nkt; ++kt) {
    __syncthreads();  // bias slice kt is visible; nobody reads the other buffer any more
    const bool more = kt + 1 < nkt;
    if (more) {  // next tile's operands and bias slice travel while this tile is computed
      load_tb(kt + 1, tbr);
      load_kv(kt + 1, kop[1], vop[1]);
    }
    tile(kt, kop[0], vop[0], tb_lds + (kt & 1) * TBBUF);
    if (more) store_tb(tbr, (kt + 1) & 1);
#pragma unroll
    for (int s = 0; s < KSQ; ++s) kop[0][s] = kop[1][s];
#pragma unroll
    for (int s = 0; s < 2; ++s) vop[0][s] = vop[1][s];
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
hipError_t launch(const TriattnFlashArgs& a, hipStream_t stream) {
  const int n_qc = (a.N + 32 * kRQ - 1) / (32 * kRQ), n_rg = (a.N + kRows - 1) / kRows;
  const long total = (long)n_qc * n_rg * a.B * a.H;
  const int per_xcd = (int)((total + 7) / 8);
  hipLaunchKernelGGL((triattn_flash_kernel<D>), dim3(per_xcd * 8), dim3(64 * kRows), 0, stream, a, n_qc, n_rg,
                     (int)total, per_xcd);
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

// Triangle-attention core (attention.py:94-135 with the two biases of tri_att.py:134-140):
//     s[q][k] = q.k + mb[i][k] + tb[h][q][k];  p = softmax_k(s);  o[q] = sum_k p[q][k] v[k]
// for every (batch, row i, head h), flash style: 32-key tiles, running maximum and sum in
// fp32, no [N][N] logits in memory.  Inputs come from the projection pass already
// multiplied by log2(e) (q also by 1/sqrt(D)), so exp() is the hardware exp2.
//
// One wave = one (b, i, h) and RQ query tiles of 32; the four waves of a work-group are
// four consecutive rows i of the same head and query range, so they read the same
// triangle-bias lines at about the same time.  All MFMA operands are loaded straight from
// global memory in operand layout (every lane reads 16 or 32 contiguous bytes):
//   S^T = K Q^T : A = K tile (row r of the tile is key rowperm16(r), so a lane ends up
//                 with 16 consecutive keys), B = Q tile (column = query)
//   O^T = V^T P^T: A = V^T (row = head channel, k = the lane-half's keys), B = P^T taken
//                 directly from the S^T accumulator registers (no cross-lane movement).
// The two biases are added in the reference's order, (q.k + mask_bias) + triangle_bias, in
// fp32: a fully masked row then degenerates to a uniform average over all real keys exactly
// as the reference's does (-1e9 absorbs the logits), and padded keys (j >= N) carry -inf.
#include "of3_device.h"
#include "of3_kernels.h"

namespace of3 {

namespace {

__device__ __forceinline__ float xhalf(float v) { return __shfl_xor(v, 32, 64); }

template <int D, int RQ>
__global__ __launch_bounds__(256) void triattn_flash_kernel(TriattnFlashArgs p) {
  constexpr int H = 4;
  constexpr int HD = H * D;
  constexpr int KSQ = D / 16;  // k-steps of the q.k product

  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63, l32 = lane & 31, lh = lane >> 5;
  const int N = p.N, Jp = p.Jp;
  const int i = blockIdx.y * 4 + wave;
  if (i >= N) return;  // no LDS, no barriers: a wave may leave early
  const int b = blockIdx.z / H, h = blockIdx.z % H;
  const int q0 = blockIdx.x * (32 * RQ);

  const size_t bih = ((size_t)b * N + i) * H + h;
  const bf16_t* Q = p.q + bih * Jp * D;
  const bf16_t* K = p.k + bih * Jp * D;
  const bf16_t* Vt = p.vt + bih * D * Jp;
  const float* tb = p.tbias + ((size_t)b * H + h) * N * Jp;
  const float* mb = p.mbias + ((size_t)b * N + i) * Jp;

  u32x4_t qop[RQ][KSQ];
  const float* tbrow[RQ];
#pragma unroll
  for (int rq = 0; rq < RQ; ++rq) {
    int qrow = q0 + 32 * rq + l32;
    qrow = qrow < Jp ? qrow : Jp - 1;
#pragma unroll
    for (int s = 0; s < KSQ; ++s) qop[rq][s] = *reinterpret_cast<const u32x4_t*>(Q + (size_t)qrow * D + 16 * s + 8 * lh);
    const int brow = qrow < N ? qrow : N - 1;
    tbrow[rq] = tb + (size_t)brow * Jp + 16 * lh;
  }

  float m_run[RQ], l_run[RQ];
  f32x16_t oacc[RQ];
#pragma unroll
  for (int rq = 0; rq < RQ; ++rq) {
    m_run[rq] = -__builtin_inff();
    l_run[rq] = 0.f;
    oacc[rq] = zero16();
  }

  const int krow = rowperm16(l32);            // key (within the tile) this lane feeds as A row
  const int vrow = rowperm16(l32);            // head channel this lane feeds as A row of V^T
  const bool vvalid = vrow < D;
  const int nkt = (N + 31) / 32;

  for (int kt = 0; kt < nkt; ++kt) {
    const int key0 = 32 * kt;
    u32x4_t kop[KSQ], vop[2];
#pragma unroll
    for (int s = 0; s < KSQ; ++s)
      kop[s] = *reinterpret_cast<const u32x4_t*>(K + (size_t)(key0 + krow) * D + 16 * s + 8 * lh);
#pragma unroll
    for (int s2 = 0; s2 < 2; ++s2) {
      u32x4_t v = {0u, 0u, 0u, 0u};
      if (vvalid) v = *reinterpret_cast<const u32x4_t*>(Vt + (size_t)vrow * Jp + key0 + 16 * lh + 8 * s2);
      vop[s2] = v;
    }
    float mbv[16];
#pragma unroll
    for (int c4 = 0; c4 < 4; ++c4) {
      const float4 t4 = *reinterpret_cast<const float4*>(mb + key0 + 16 * lh + 4 * c4);
      mbv[4 * c4] = t4.x;
      mbv[4 * c4 + 1] = t4.y;
      mbv[4 * c4 + 2] = t4.z;
      mbv[4 * c4 + 3] = t4.w;
    }

#pragma unroll
    for (int rq = 0; rq < RQ; ++rq) {
      float tbv[16];
#pragma unroll
      for (int c4 = 0; c4 < 4; ++c4) {
        const float4 t4 = *reinterpret_cast<const float4*>(tbrow[rq] + key0 + 4 * c4);
        tbv[4 * c4] = t4.x;
        tbv[4 * c4 + 1] = t4.y;
        tbv[4 * c4 + 2] = t4.z;
        tbv[4 * c4 + 3] = t4.w;
      }
      f32x16_t s = zero16();
#pragma unroll
      for (int ks = 0; ks < KSQ; ++ks) s = mfma_32x32x16(kop[ks], qop[rq][ks], s);

      float mx = -__builtin_inff();
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        s[v] = (s[v] + mbv[v]) + tbv[v];
        mx = fmaxf(mx, s[v]);
      }
      mx = fmaxf(mx, xhalf(mx));
      const float m_new = fmaxf(m_run[rq], mx);
      const float alpha = fast_exp2(m_run[rq] - m_new);
      float pr[16];
      float rs = 0.f;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        pr[v] = fast_exp2(s[v] - m_new);
        rs += pr[v];
      }
      rs += xhalf(rs);
      l_run[rq] = l_run[rq] * alpha + rs;
      m_run[rq] = m_new;
#pragma unroll
      for (int v = 0; v < 16; ++v) oacc[rq][v] *= alpha;
      u32x4_t pop[2];
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
        for (int w = 0; w < 4; ++w) pop[s2][w] = pack_bf16(pr[8 * s2 + 2 * w], pr[8 * s2 + 2 * w + 1]);
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2) oacc[rq] = mfma_32x32x16(vop[s2], pop[s2], oacc[rq]);
    }
  }

  // ---- finalize: lane (query l32, half lh) owns head channels 16*lh + v
  if (16 * lh < D) {
#pragma unroll
    for (int rq = 0; rq < RQ; ++rq) {
      const int qrow = q0 + 32 * rq + l32;
      if (qrow >= N) continue;
      const float inv = fast_rcp(l_run[rq]);
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

template <int D, int RQ>
hipError_t launch(const TriattnFlashArgs& a, hipStream_t stream) {
  const dim3 grid((a.N + 32 * RQ - 1) / (32 * RQ), (a.N + 3) / 4, a.B * a.H);
  hipLaunchKernelGGL((triattn_flash_kernel<D, RQ>), grid, dim3(256), 0, stream, a);
  return hipGetLastError();
}

}  // namespace

hipError_t triattn_flash_launch(const TriattnFlashArgs& args, int D, hipStream_t stream) {
  if (args.H != 4) return hipErrorInvalidValue;
  if (D == 32) return launch<32, 4>(args, stream);
  if (D == 16) return launch<16, 4>(args, stream);
  return hipErrorInvalidValue;
}

}  // namespace of3

// Single-representation attention with pair bias, the trunk's AttentionPairBias
// (attention_pair_bias.py:189-244 with Attention._prep_qkv / _attention / _wrap_up,
// attention.py:265-302, :94-135), once per PairFormerBlock (pairformer.py:189-201):
//     an = LN(a);  q = (an Wq^T + bq) / sqrt(D), k = an Wk^T, v = an Wv^T      (H heads of width D)
//     s[h][q][k] = q.k + inf * (mask[k] - 1) + pair_bias[h][q][k];  p = softmax_k(s);  o = p v
//     out = [a +] (o * sigmoid(an Wg^T)) Wo^T
// The pair bias [B][H][N][N] is the output of the pair-bias projection kernel.  With N tokens of
// c_s = 384 channels the whole module is about 2 GFLOP at N = 768: three small kernels.
//
//  1. single_proj: a work-group normalises 32 positions into an LDS tile [position][channel]
//     (bf16, 16-byte chunks XOR-swizzled by the position) and its waves compute 32-wide output
//     tiles with K = c_s MFMA steps, the weights read straight from global memory (they stay in
//     L2).  A tile is one head of one of q, k, v, g, padded from D = 24 to 32 channels with zero
//     weight rows, so q and k come out as [B][H][Np][32] with zero padding.  For q, k and g the
//     weights are the A operand (rows dealt by rowperm16: a lane ends up with 16 consecutive
//     channels of one position); for v the positions are the A operand, so that a lane holds one
//     channel of 4-position runs and V^T [B][H][32][Np] is written with 8-byte stores.
//     q carries log2(e) / sqrt(D) (the softmax below uses exp2), g is stored after the sigmoid.
//     The first padding channel (index D) carries the key mask: q gets 1 there and k gets
//     inf * (mask[key] - 1) * log2(e), or -inf for the rows between N and Np, so the q.k
//     product itself adds the mask bias and gives padded keys a weight of exactly zero.
//  2. single_attn: one work-group per (batch, head, 32 queries), its four waves splitting the key
//     tiles and merging their partial softmaxes through LDS at the end; flash style over 32-key tiles:
//     S^T = K Q^T with the accumulator initialised to pair bias * log2(e), the next tile's
//     operands requested before the current tile's arithmetic, running
//     maximum and sum in fp32, O^T = V^T P^T with P^T taken from the S^T registers; the result
//     is divided by the sum, multiplied by the gate and written as [B][N][H*D].
//  3. single_out: the same tiling as 1 without the LayerNorm: out = [a +] og Wo^T.
#include "of3_device.h"
#include "of3_kernels.h"
#include "of3_rowtile.h"

namespace of3 {

namespace {

using namespace rowtile;

constexpr int kDP = 32;          // head width padded to one MFMA tile

// ---- 1. LayerNorm + q, k, v, g ------------------------------------------------------------
__global__ __launch_bounds__(256) void single_proj_kernel(SingleAttnArgs p) {
  __shared__ u32x4_t act[32 * kChunks];
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63, l32 = lane & 31, lh = lane >> 5;
  const int N = p.N, Np = p.Np, H = p.H, D = p.D;
  const int b = blockIdx.z;
  const long pos0 = (long)blockIdx.x * 32;
  fill_tile<true>(act, p.a + (size_t)b * N * kK, kK, pos0, N, p.ln_w, p.ln_b, wave, lane);
  __syncthreads();

  const long pos = pos0 + l32;  // position of this lane in the weights-are-A tiles
  const float q_scale = kLog2e * __builtin_amdgcn_rsqf((float)D);
  for (int tile = blockIdx.y * 4 + wave; tile < 4 * H; tile += gridDim.y * 4) {
    const int kind = tile / H, h = tile - kind * H;  // 0 q, 1 k, 2 v, 3 g
    if (kind != 2) {
      const bf16_t* W = kind == 0 ? p.wq : (kind == 1 ? p.wk : p.wg);
      const int dch = rowperm16(l32);
      const f32x16_t acc = tile_product<true>(act, dch < D ? W + (size_t)(h * D + dch) * kK : nullptr, l32, lh);
      // lane (position, half lh): padded channels 16*lh + v
      float f[16];
#pragma unroll
      for (int v = 0; v < 16; ++v) f[v] = acc[v];
      if (kind == 0) {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int d = 16 * lh + v;
          f[v] = d < D ? (f[v] + bf16_to_f32(p.bq[h * D + d])) * q_scale : (d == D ? 1.f : 0.f);
        }
      } else if (kind == 1) {
        // the key's mask bias rides in the first padding channel (q holds 1 there)
        float mb = 0.f;
        if (pos >= N) mb = -__builtin_inff();
        else if (p.mask) mb = p.inf * kLog2e * (p.mask[(size_t)b * N + pos] - 1.f);
#pragma unroll
        for (int v = 0; v < 16; ++v)
          if (16 * lh + v == D) f[v] = mb;
      } else if (kind == 3) {
#pragma unroll
        for (int v = 0; v < 16; ++v) f[v] = sigmoidf_fast(f[v]);
      }
      u32x4_t o0, o1;
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        o0[w] = pack_bf16(f[2 * w], f[2 * w + 1]);
        o1[w] = pack_bf16(f[8 + 2 * w], f[8 + 2 * w + 1]);
      }
      if (kind == 3) {
        if (pos < N) {
          bf16_t* dst = p.g + ((size_t)b * N + pos) * (H * D) + h * D + 16 * lh;
          if (16 * lh < D) *reinterpret_cast<u32x4_t*>(dst) = o0;
          if (16 * lh + 8 < D) *reinterpret_cast<u32x4_t*>(dst + 8) = o1;
        }
      } else if (pos < Np) {
        bf16_t* dst = (kind == 0 ? p.q : p.k) + (((size_t)b * H + h) * Np + pos) * kDP + 16 * lh;
        *reinterpret_cast<u32x4_t*>(dst) = o0;
        *reinterpret_cast<u32x4_t*>(dst + 8) = o1;
      }
    } else {
      const f32x16_t acc = tile_product<false>(act, l32 < D ? p.wv + (size_t)(h * D + l32) * kK : nullptr, l32, lh);
      // lane (padded channel l32, half lh): positions pos0 + 8*(v/4) + 4*lh + (v%4)
      bf16_t* row = p.vt + (((size_t)b * H + h) * kDP + l32) * Np;
#pragma unroll
      for (int g4 = 0; g4 < 4; ++g4) {
        const long pp = pos0 + 8 * g4 + 4 * lh;
        if (pp < Np) {
          float f[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) f[e] = pp + e < N ? acc[4 * g4 + e] : 0.f;  // padded keys: zeros
          u32x2_t o = {pack_bf16(f[0], f[1]), pack_bf16(f[2], f[3])};
          *reinterpret_cast<u32x2_t*>(row + pp) = o;
        }
      }
    }
  }
}

// ---- 2. attention core -------------------------------------------------------------------
constexpr int kSplit = 4;  // waves sharing one (batch, head, 32 queries)

__global__ __launch_bounds__(64 * kSplit) void single_attn_kernel(SingleAttnArgs p, int q_tiles) {
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63, l32 = lane & 31, lh = lane >> 5;
  const int N = p.N, Np = p.Np, H = p.H, D = p.D;
  // the kSplit waves of a work-group share one (batch, head, 32 queries) and split its key tiles
  // (wave w takes tiles w, w+kSplit, ...): a single wave walking all tiles is bound by the latency of
  // its own MFMA -> softmax -> MFMA chain, and the problem offers few waves otherwise
  __shared__ float merge[kSplit][18][64];
  const int qt = blockIdx.x;
  const int h = blockIdx.y, b = blockIdx.z;
  const int q0 = qt * 32;
  int qrow = q0 + l32;
  const bool q_valid = qrow < N;
  qrow = q_valid ? qrow : N - 1;

  const size_t bh = (size_t)b * H + h;
  const bf16_t* Q = p.q + (bh * Np + qrow) * kDP;
  const bf16_t* K = p.k + bh * Np * kDP;
  const bf16_t* Vt = p.vt + bh * kDP * Np;
  const bf16_t* pb_row = p.pair_bias + (bh * N + qrow) * N;
  const bool vec_ok = (N % 8) == 0;  // 16-byte aligned runs of the bias rows

  u32x4_t qop[2];
#pragma unroll
  for (int s = 0; s < 2; ++s) qop[s] = *reinterpret_cast<const u32x4_t*>(Q + 16 * s + 8 * lh);
  const int krow = rowperm16(l32);

  // operands of one key tile: K rows dealt by rowperm16 (a lane ends up with keys k0 + 16*lh + v);
  // V^T rows = padded channels dealt by rowperm16, lane-half lh and k-step s2 feed keys
  // 16*lh + 8*s2 .. +7, the keys registers 8*s2 .. 8*s2+7 of that lane-half hold in S^T; the
  // lane's 16 pair-bias values
  auto load_tile = [&](int kt, u32x4_t (&kc)[2], u32x4_t (&vc)[2], u32x4_t (&braw)[2]) {
    const int k0 = 32 * kt;
#pragma unroll
    for (int s = 0; s < 2; ++s) kc[s] = *reinterpret_cast<const u32x4_t*>(K + (size_t)(k0 + krow) * kDP + 16 * s + 8 * lh);
#pragma unroll
    for (int s2 = 0; s2 < 2; ++s2) vc[s2] = *reinterpret_cast<const u32x4_t*>(Vt + (size_t)krow * Np + k0 + 16 * lh + 8 * s2);
    load16_raw(pb_row, k0 + 16 * lh, N, vec_ok, braw);
  };

  float m_run = -__builtin_inff(), l_run = 0.f;
  f32x16_t oacc = zero16();
  const int nkt = (N + 31) / 32;
  u32x4_t kn[2], vn[2], bn[2];
  if (wave < nkt) load_tile(wave, kn, vn, bn);
  for (int kt = wave; kt < nkt; kt += kSplit) {
    u32x4_t kc[2], vc[2], braw[2];
#pragma unroll
    for (int s = 0; s < 2; ++s) kc[s] = kn[s], vc[s] = vn[s], braw[s] = bn[s];
    if (kt + kSplit < nkt) load_tile(kt + kSplit, kn, vn, bn);  // in flight under this tile's arithmetic

    f32x16_t s;
#pragma unroll
    for (int w = 0; w < 8; ++w) {
      s[2 * w] = bf16_lo(braw[w >> 2][w & 3]) * kLog2e;
      s[2 * w + 1] = bf16_hi(braw[w >> 2][w & 3]) * kLog2e;
    }
    s = mfma_32x32x16(kc[0], qop[0], s);
    s = mfma_32x32x16(kc[1], qop[1], s);  // includes the mask bias (-inf for keys past N)

    float mx = s[0];
#pragma unroll
    for (int v = 1; v < 16; ++v) mx = fmaxf(mx, s[v]);
    const float m_new = fmaxf(m_run, fmaxf(mx, xhalf(mx)));  // every tile holds at least one real key
    const float alpha = fast_exp2(m_run - m_new);            // exp2(-inf) = 0 on the first tile
    l_run *= alpha;
#pragma unroll
    for (int v = 0; v < 16; ++v) oacc[v] *= alpha;
    m_run = m_new;
    u32x4_t pop[2];
    float rs = 0.f;
#pragma unroll
    for (int w = 0; w < 8; ++w) {
      const uint32_t pk = pack_bf16(fast_exp2(s[2 * w] - m_new), fast_exp2(s[2 * w + 1] - m_new));
      rs += bf16_lo(pk) + bf16_hi(pk);  // the sum of the weights the P V product uses
      pop[w >> 2][w & 3] = pk;
    }
    l_run += rs;
    oacc = mfma_32x32x16(vc[0], pop[0], oacc);
    oacc = mfma_32x32x16(vc[1], pop[1], oacc);
  }

  // ---- merge the partial softmaxes: common maximum, rescaled sums and accumulators
  merge[wave][16][lane] = m_run;  // -inf for a wave without tiles
  merge[wave][17][lane] = l_run + xhalf(l_run);
#pragma unroll
  for (int v = 0; v < 16; ++v) merge[wave][v][lane] = oacc[v];
  __syncthreads();
  if (wave != 0) return;
  float m_tot = merge[0][16][lane];  // wave 0 always has tile 0: finite
#pragma unroll
  for (int w = 1; w < kSplit; ++w) m_tot = fmaxf(m_tot, merge[w][16][lane]);
  float l_tot = 0.f;
#pragma unroll
  for (int v = 0; v < 16; ++v) oacc[v] = 0.f;
#pragma unroll
  for (int w = 0; w < kSplit; ++w) {
    const float sc = fast_exp2(merge[w][16][lane] - m_tot);  // 0 for a wave without tiles
    l_tot += merge[w][17][lane] * sc;
#pragma unroll
    for (int v = 0; v < 16; ++v) oacc[v] += merge[w][v][lane] * sc;
  }

  // lane (query l32, half lh) owns head channels 16*lh + v
  const float inv = fast_rcp(l_tot);
  if (q_valid && 16 * lh < D) {
    const size_t off = ((size_t)b * N + qrow) * (H * D) + h * D + 16 * lh;
    u32x4_t graw[2];
    load16_raw(p.g + off, 0, D - 16 * lh, true, graw);
    u32x4_t o0, o1;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      o0[w] = pack_bf16(oacc[2 * w] * inv * bf16_lo(graw[0][w]), oacc[2 * w + 1] * inv * bf16_hi(graw[0][w]));
      o1[w] = pack_bf16(oacc[8 + 2 * w] * inv * bf16_lo(graw[1][w]), oacc[8 + 2 * w + 1] * inv * bf16_hi(graw[1][w]));
    }
    bf16_t* dst = p.og + off;
    *reinterpret_cast<u32x4_t*>(dst) = o0;
    if (16 * lh + 8 < D) *reinterpret_cast<u32x4_t*>(dst + 8) = o1;
  }
}

// ---- 3. output projection ----------------------------------------------------------------
__global__ __launch_bounds__(256) void single_out_kernel(SingleAttnArgs p) {
  __shared__ u32x4_t act[32 * kChunks];
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63, l32 = lane & 31, lh = lane >> 5;
  const int N = p.N;
  const int b = blockIdx.z;
  const long pos0 = (long)blockIdx.x * 32;
  fill_tile<false>(act, p.og + (size_t)b * N * kK, kK, pos0, N, nullptr, nullptr, wave, lane);
  __syncthreads();
  const long pos = pos0 + l32;
  for (int tile = blockIdx.y * 4 + wave; tile < kK / 32; tile += gridDim.y * 4) {
    const f32x16_t acc = tile_product<true>(act, p.wo + (size_t)(32 * tile + rowperm16(l32)) * kK, l32, lh);
    if (pos < N) {
      const size_t off = ((size_t)b * N + pos) * kK + 32 * tile + 16 * lh;
      float f[16];
#pragma unroll
      for (int v = 0; v < 16; ++v) f[v] = acc[v];
      if (p.add_residual) {
        // the reference adds the module's bf16 output to s: round before the add
        u32x4_t r[2];
        load16_raw(p.a + off, 0, 16, true, r);
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
}

}  // namespace

hipError_t single_attn_launch(const SingleAttnArgs& a, hipStream_t stream) {
  if (a.H * a.D != kK || a.D >= kDP || (a.D % 8) != 0 || a.H < 1 || a.N < 1 || a.B < 1 || a.B > 65535 || a.H > 65535)
    return hipErrorInvalidValue;
  if (a.Np != (a.N + 31) / 32 * 32) return hipErrorInvalidValue;
  const int row_blocks = a.Np / 32;
  hipLaunchKernelGGL(single_proj_kernel, dim3(row_blocks, a.H, a.B), dim3(256), 0, stream, a);  // one tile per wave
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(single_attn_kernel, dim3(row_blocks, a.H, a.B), dim3(64 * kSplit), 0, stream, a, row_blocks);
  e = hipGetLastError();
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(single_out_kernel, dim3(row_blocks, 3, a.B), dim3(256), 0, stream, a);
  return hipGetLastError();
}

}  // namespace of3

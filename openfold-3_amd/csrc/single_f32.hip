// fp32 versions of the single-representation kernels (AttentionPairBias of the trunk,
// attention_pair_bias.py:189-244, and the SwiGLU transition over s, transition.py:225-271): plain
// fp32 FMA arithmetic in the reference's order of operations, any N, C_s <= 512, head width
// <= 64, hidden width <= 2048.  The precision path, not a fast one: the linear layers give a thread
// one output channel and stage the weights through LDS, the attention gives a thread one query.
#include "of3_device.h"
#include "of3_kernels.h"
#include "of3_launch.h"

namespace of3 {

namespace {

constexpr int kRows = 4;        // positions per work-group (one wave normalises one row)
constexpr int kThreads = 256;
constexpr int kMaxCs = 512;
constexpr int kMaxHidden = 2048;
constexpr float kEps = 1e-5f;

__device__ __forceinline__ float wave_sum_f32(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
__device__ __forceinline__ float sigmoid_f32(float x) { return 1.0f / (1.0f + expf(-x)); }

// ---- linear layers over kRows rows held in LDS -----------------------------------------------------
// y[r][o] = sum_k xs[r][k] W[o][k], k ascending, one fused multiply-add per term.  Thread t owns output
// o0 + t of a tile of kThreads outputs.  The weights of a tile come through LDS in pieces of kWK inputs:
// 16 lanes read 256 contiguous bytes of a weight row (a thread walking its own row would touch 64
// cache lines per wave instruction), the piece is stored with a row stride of kWK + 1 words, so that
// both the staging stores and the per-thread row reads are free of bank conflicts, and the next piece
// is already on its way in registers while the current one is multiplied.  xs must be readable and
// zero up to the next multiple of kWK past K: whole pieces are multiplied, the padding adds zeros.
constexpr int kWK = 64;
constexpr int kWLd = kWK + 1;
constexpr int kWLoads = kWK / 4;  // 16-byte pieces per thread and tile piece (kThreads rows of kWK / 4 pieces)
constexpr size_t kWTileBytes = (size_t)kThreads * kWLd * sizeof(float);

__device__ __forceinline__ int round_up_wk(int n) { return (n + kWK - 1) / kWK * kWK; }

template <bool VEC, int LD, class Epilogue>
__device__ __forceinline__ void rows_linear_impl(const float (*xs)[LD], const float* __restrict__ W, int n_out, int K,
                                                 float* wt, Epilogue&& epilogue) {
  const int t = threadIdx.x;
  for (int o0 = 0; o0 < n_out; o0 += kThreads) {
    float4 nxt[kWLoads];
    // every load is issued whatever the lane's position: addresses are clamped into the matrix, and
    // what lies outside is masked to zero bit-wise when the piece goes to LDS, after the products of
    // the piece before (a load or a replacement under a lane condition makes the compiler wait for all
    // loads in flight where the lanes join, and a mask applied here would wait for them at once)
    auto fetch = [&](int k0) {
#pragma unroll
      for (int i = 0; i < kWLoads; ++i) {
        const int idx = t + i * kThreads, row = idx >> 4, k = k0 + 4 * (idx & 15), o = o0 + row;
        const float* src = W + (size_t)(o < n_out ? o : n_out - 1) * K;
        if (VEC) {  // K is a multiple of 4: a piece lies inside the row or outside
          nxt[i] = *reinterpret_cast<const float4*>(src + (k < K ? k : K - 4));
        } else {
          nxt[i].x = src[k < K ? k : K - 1];
          nxt[i].y = src[k + 1 < K ? k + 1 : K - 1];
          nxt[i].z = src[k + 2 < K ? k + 2 : K - 1];
          nxt[i].w = src[k + 3 < K ? k + 3 : K - 1];
        }
      }
    };
    auto to_lds = [&](int k0) {
#pragma unroll
      for (int i = 0; i < kWLoads; ++i) {
        const int idx = t + i * kThreads, row = idx >> 4, k = k0 + 4 * (idx & 15), o = o0 + row;
        float* dst = wt + row * kWLd + 4 * (idx & 15);
        const float v[4] = {nxt[i].x, nxt[i].y, nxt[i].z, nxt[i].w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const unsigned keep = o < n_out && k + (VEC ? 0 : j) < K ? ~0u : 0u;
          dst[j] = __uint_as_float(__float_as_uint(v[j]) & keep);
        }
      }
    };
    float acc[kRows];
#pragma unroll
    for (int r = 0; r < kRows; ++r) acc[r] = 0.f;
    fetch(0);
    for (int k0 = 0; k0 < K; k0 += kWK) {
      __syncthreads();  // the previous piece has been multiplied by everybody
      to_lds(k0);
      __syncthreads();
      if (k0 + kWK < K) fetch(k0 + kWK);
      const float* wrow = wt + t * kWLd;
#pragma unroll 4
      for (int kk = 0; kk < kWK; kk += 4) {
        const float w0 = wrow[kk], w1 = wrow[kk + 1], w2 = wrow[kk + 2], w3 = wrow[kk + 3];
#pragma unroll
        for (int r = 0; r < kRows; ++r) {
          const float4 x = *reinterpret_cast<const float4*>(&xs[r][k0 + kk]);  // one address per wave: a broadcast
          acc[r] = fmaf(x.x, w0, acc[r]);
          acc[r] = fmaf(x.y, w1, acc[r]);
          acc[r] = fmaf(x.z, w2, acc[r]);
          acc[r] = fmaf(x.w, w3, acc[r]);
        }
      }
    }
    if (o0 + t < n_out) epilogue(o0 + t, acc);
  }
}
template <int LD, class Epilogue>
__device__ __forceinline__ void rows_linear(const float (*xs)[LD], const float* __restrict__ W, int n_out, int K,
                                            float* wt, Epilogue&& epilogue) {
  if ((K & 3) == 0 && (reinterpret_cast<uintptr_t>(W) & 15u) == 0) rows_linear_impl<true>(xs, W, n_out, K, wt, epilogue);
  else rows_linear_impl<false>(xs, W, n_out, K, wt, epilogue);
}

// LayerNorm of rows pos0 .. pos0+kRows-1 of src [rows][C] into xn (two-pass statistics); rows
// past n_rows give zeros, and so do the channels from C to the next multiple of kWK
__device__ __forceinline__ void norm_rows(const float* __restrict__ src, long pos0, long n_rows, int C,
                                          const float* __restrict__ w, const float* __restrict__ b,
                                          float (*xn)[kMaxCs]) {
  const int r = threadIdx.x >> 6, l = threadIdx.x & 63;
  const long row = pos0 + r;
  const float* x = row < n_rows ? src + row * C : nullptr;
  float s = 0.f;
  if (x)
    for (int c = l; c < C; c += 64) s += x[c];
  const float mean = wave_sum_f32(s) / (float)C;
  float q = 0.f;
  if (x)
    for (int c = l; c < C; c += 64) {
      const float d = x[c] - mean;
      q += d * d;
    }
  const float rstd = 1.0f / sqrtf(wave_sum_f32(q) / (float)C + kEps);
  for (int c = l; c < round_up_wk(C); c += 64) xn[r][c] = x && c < C ? (x[c] - mean) * rstd * w[c] + b[c] : 0.f;
}

// q (bias added, then / sqrt(D)), k, v and the gate after the sigmoid, all [B*N][H*D]
__global__ __launch_bounds__(kThreads) void single_proj_f32(SingleAttnF32Args p) {
  __shared__ __align__(16) float xn[kRows][kMaxCs];
  extern __shared__ float wt[];
  const long rows = (long)p.B * p.N, pos0 = (long)blockIdx.x * kRows;
  const int C = p.C, HD = p.H * p.D;
  norm_rows(p.a, pos0, rows, C, p.ln_w, p.ln_b, xn);
  const float scale = 1.0f / sqrtf((float)p.D);
  for (int kind = 0; kind < 4; ++kind) {
    const float* W = kind == 0 ? p.wq : kind == 1 ? p.wk : kind == 2 ? p.wv : p.wg;
    float* dst = kind == 0 ? p.q : kind == 1 ? p.k : kind == 2 ? p.v : p.g;
    rows_linear(xn, W, HD, C, wt, [&](int ch, const float (&acc)[kRows]) {
#pragma unroll
      for (int r = 0; r < kRows; ++r) {
        if (pos0 + r >= rows) continue;
        float v = acc[r];
        if (kind == 0) v = (v + p.bq[ch]) * scale;
        if (kind == 3) v = sigmoid_f32(v);
        dst[(pos0 + r) * HD + ch] = v;
      }
    });
  }
}

// 32 queries of one (batch, head) per work-group, four threads per query: keys in chunks of 32 through
// LDS together with the [32 queries][32 keys] slice of the pair bias, thread (query, part) takes keys
// 8 part .. 8 part + 7 of every chunk with a running softmax of its own; the four partial results of a
// query are merged at the end; output times gate
constexpr int kAttnQ = 32, kAttnParts = 4;
template <int DMAX>
__global__ __launch_bounds__(kAttnQ * kAttnParts) void single_attn_f32(SingleAttnF32Args p) {
  constexpr int KC = 32, KP = KC / kAttnParts, NT = kAttnQ * kAttnParts;
  __shared__ float ks[KC][DMAX], vs[KC][DMAX], mbs[KC];
  __shared__ float pbs[kAttnQ][KC + 1];
  __shared__ float part_o[kAttnParts][kAttnQ][DMAX + 1], part_m[kAttnParts][kAttnQ], part_l[kAttnParts][kAttnQ];
  const int N = p.N, H = p.H, D = p.D, HD = H * D;
  const int qg = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  const int ql = threadIdx.x % kAttnQ, part = threadIdx.x / kAttnQ;
  const int qi = qg * kAttnQ + ql;
  const bool active = qi < N;
  float qv[DMAX], ov[DMAX];
#pragma unroll
  for (int d = 0; d < DMAX; ++d) {
    qv[d] = (active && d < D) ? p.q[((size_t)b * N + qi) * HD + h * D + d] : 0.f;
    ov[d] = 0.f;
  }
  const float* pb = p.pair_bias + (((size_t)b * H + h) * N + (size_t)qg * kAttnQ) * N;
  const float ninf = -__builtin_inff();
  float m = ninf, l = 0.f;
  for (int k0 = 0; k0 < N; k0 += KC) {
    __syncthreads();
    for (int e = threadIdx.x; e < KC * DMAX; e += NT) {
      const int kk = e / DMAX, d = e % DMAX;
      const bool in = k0 + kk < N && d < D;
      ks[kk][d] = in ? p.k[((size_t)b * N + k0 + kk) * HD + h * D + d] : 0.f;
      vs[kk][d] = in ? p.v[((size_t)b * N + k0 + kk) * HD + h * D + d] : 0.f;
    }
    for (int e = threadIdx.x; e < kAttnQ * KC; e += NT) {
      const int r = e / KC, c = e % KC;
      pbs[r][c] = (qg * kAttnQ + r < N && k0 + c < N) ? pb[(size_t)r * N + k0 + c] : 0.f;
    }
    if (threadIdx.x < KC) {
      const int kx = k0 + threadIdx.x;
      float mv = 1.f;
      if (kx < N && p.mask) mv = p.mask[(size_t)b * N + kx];
      mbs[threadIdx.x] = p.inf * (mv - 1.f);
    }
    __syncthreads();
    const int kn = N - k0 < KC ? N - k0 : KC;
    float s[KP];
    float cmax = ninf;
#pragma unroll
    for (int j = 0; j < KP; ++j) {
      const int kk = part * KP + j;
      float acc = 0.f;
#pragma unroll
      for (int d = 0; d < DMAX; ++d) acc = fmaf(qv[d], ks[kk][d], acc);
      // logits in the reference's order: q.k, then the mask bias, then the pair bias
      acc = acc + mbs[kk];
      acc = acc + pbs[ql][kk];
      s[j] = kk < kn ? acc : ninf;
      cmax = fmaxf(cmax, s[j]);
    }
    if (cmax == ninf) continue;  // none of this thread's keys of the chunk exists (the barriers are above)
    const float m_new = fmaxf(m, cmax);
    const float alpha = expf(m - m_new);  // 0 the first time (m = -inf, m_new finite)
    l *= alpha;
#pragma unroll
    for (int d = 0; d < DMAX; ++d) ov[d] *= alpha;
#pragma unroll
    for (int j = 0; j < KP; ++j) {
      const float pw = expf(s[j] - m_new);  // 0 for a key that does not exist
      l += pw;
#pragma unroll
      for (int d = 0; d < DMAX; ++d) ov[d] = fmaf(pw, vs[part * KP + j][d], ov[d]);
    }
    m = m_new;
  }
  // merge the parts of a query: a part that saw no key has m = -inf, l = 0 and weighs nothing
  part_m[part][ql] = m;
  part_l[part][ql] = l;
#pragma unroll
  for (int d = 0; d < DMAX; ++d) part_o[part][ql][d] = ov[d];
  __syncthreads();
  if (part == 0 && active) {
    float mm = ninf;
#pragma unroll
    for (int q = 0; q < kAttnParts; ++q) mm = fmaxf(mm, part_m[q][ql]);
    float lsum = 0.f;
#pragma unroll
    for (int d = 0; d < DMAX; ++d) ov[d] = 0.f;
#pragma unroll
    for (int q = 0; q < kAttnParts; ++q) {
      const float w = part_m[q][ql] == ninf ? 0.f : expf(part_m[q][ql] - mm);
      lsum = fmaf(part_l[q][ql], w, lsum);
#pragma unroll
      for (int d = 0; d < DMAX; ++d) ov[d] = fmaf(part_o[q][ql][d], w, ov[d]);
    }
    const float inv = 1.0f / lsum;
    const size_t off = ((size_t)b * N + qi) * HD + h * D;
#pragma unroll
    for (int d = 0; d < DMAX; ++d)
      if (d < D) p.og[off + d] = (ov[d] * inv) * p.g[off + d];
  }
}

__global__ __launch_bounds__(kThreads) void single_out_f32(SingleAttnF32Args p) {
  __shared__ __align__(16) float og[kRows][kMaxCs];
  extern __shared__ float wt[];
  const long rows = (long)p.B * p.N, pos0 = (long)blockIdx.x * kRows;
  const int C = p.C, HD = p.H * p.D, hd_pad = round_up_wk(HD);
  for (int idx = threadIdx.x; idx < kRows * hd_pad; idx += kThreads) {
    const int r = idx / hd_pad, c = idx % hd_pad;
    og[r][c] = pos0 + r < rows && c < HD ? p.og[(pos0 + r) * HD + c] : 0.f;
  }
  rows_linear(og, p.wo, C, HD, wt, [&](int o, const float (&acc)[kRows]) {
#pragma unroll
    for (int r = 0; r < kRows; ++r) {
      if (pos0 + r >= rows) continue;
      float v = acc[r];
      if (p.add_residual) v = p.a[(pos0 + r) * C + o] + v;
      p.out[(pos0 + r) * C + o] = v;
    }
  });
}

// out = [x +] ((silu(LN(x) Wa^T) * (LN(x) Wb^T)) Wout^T) * mask for kRows rows per work-group; the
// hidden activations stay in LDS
__global__ __launch_bounds__(kThreads) void row_transition_f32(RowTransitionF32Args p) {
  __shared__ __align__(16) float xn[kRows][kMaxCs];
  __shared__ __align__(16) float hid[kRows][kMaxHidden];
  extern __shared__ float wt[];
  const long pos0 = (long)blockIdx.x * kRows;
  const int C = p.C, HID = p.HID;
  norm_rows(p.x, pos0, p.rows, C, p.ln_w, p.ln_b, xn);
  for (int idx = HID + threadIdx.x; idx < round_up_wk(HID); idx += kThreads)
#pragma unroll
    for (int r = 0; r < kRows; ++r) hid[r][idx] = 0.f;
  // a thread writes a and then silu(a) * b into the same words of hid: no barrier between the two
  rows_linear(xn, p.wa, HID, C, wt, [&](int o, const float (&acc)[kRows]) {
#pragma unroll
    for (int r = 0; r < kRows; ++r) hid[r][o] = acc[r];
  });
  rows_linear(xn, p.wb, HID, C, wt, [&](int o, const float (&acc)[kRows]) {
#pragma unroll
    for (int r = 0; r < kRows; ++r) {
      const float a = hid[r][o];
      hid[r][o] = (a * sigmoid_f32(a)) * acc[r];  // silu(a) * b (activations.py:60-61)
    }
  });
  rows_linear(hid, p.wout, C, HID, wt, [&](int o, const float (&acc)[kRows]) {
#pragma unroll
    for (int r = 0; r < kRows; ++r) {
      if (pos0 + r >= p.rows) continue;
      float v = acc[r];
      if (p.mask) v = v * p.mask[pos0 + r];
      if (p.add_residual) v = p.x[(pos0 + r) * C + o] + v;
      p.out[(pos0 + r) * C + o] = v;
    }
  });
}

}  // namespace

hipError_t single_attn_fwd_f32(const SingleAttnF32Args& a, hipStream_t stream) {
  if (a.C < 1 || a.C > kMaxCs || a.H < 1 || a.D < 1 || a.D > 64 || a.H * a.D > kMaxCs || a.N < 1 || a.B < 1 ||
      a.B > 65535 || a.H > 65535)
    return hipErrorInvalidValue;
  const long rows = (long)a.B * a.N;
  const long blocks = (rows + kRows - 1) / kRows;
  if (blocks > 0x7fffffffl) return hipErrorInvalidValue;
  hipError_t e = allow_dynamic_lds<single_proj_f32>(kWTileBytes);
  if (e == hipSuccess) e = allow_dynamic_lds<single_out_f32>(kWTileBytes);
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(single_proj_f32, dim3((unsigned)blocks), dim3(kThreads), kWTileBytes, stream, a);
  e = hipGetLastError();
  if (e != hipSuccess) return e;
  const dim3 grid((a.N + kAttnQ - 1) / kAttnQ, a.H, a.B);
  if (a.D <= 32) hipLaunchKernelGGL(single_attn_f32<32>, grid, dim3(kAttnQ * kAttnParts), 0, stream, a);
  else hipLaunchKernelGGL(single_attn_f32<64>, grid, dim3(kAttnQ * kAttnParts), 0, stream, a);
  e = hipGetLastError();
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(single_out_f32, dim3((unsigned)blocks), dim3(kThreads), kWTileBytes, stream, a);
  return hipGetLastError();
}

hipError_t row_transition_fwd_f32(const RowTransitionF32Args& a, hipStream_t stream) {
  if (a.rows < 1 || a.C < 1 || a.C > kMaxCs || a.HID < 1 || a.HID > kMaxHidden) return hipErrorInvalidValue;
  const long blocks = (a.rows + kRows - 1) / kRows;
  if (blocks > 0x7fffffffl) return hipErrorInvalidValue;
  const hipError_t e = allow_dynamic_lds<row_transition_f32>(kWTileBytes);
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(row_transition_f32, dim3((unsigned)blocks), dim3(kThreads), kWTileBytes, stream, a);
  return hipGetLastError();
}

}  // namespace of3

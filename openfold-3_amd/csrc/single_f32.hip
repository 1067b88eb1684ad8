// fp32 versions of the single-representation kernels (AttentionPairBias of the trunk,
// attention_pair_bias.py:189-244, and the SwiGLU transition over s, transition.py:225-271): plain
// fp32 FMA arithmetic in the reference's order of operations, any N, C_s <= 512, head width
// <= 64, hidden width <= 2048.  The precision path, not a fast one.
#include "of3_device.h"
#include "of3_kernels.h"

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
__device__ __forceinline__ float dot_f32(const float* __restrict__ x, const float* __restrict__ w, int n) {
  float acc = 0.f;
  for (int k = 0; k < n; ++k) acc = fmaf(x[k], w[k], acc);
  return acc;
}

// LayerNorm of rows pos0 .. pos0+kRows-1 of src [rows][C] into xn (two-pass statistics); rows
// past n_rows give zeros
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
  for (int c = l; c < C; c += 64) xn[r][c] = x ? (x[c] - mean) * rstd * w[c] + b[c] : 0.f;
}

// q (bias added, then / sqrt(D)), k, v and the gate after the sigmoid, all [B*N][H*D]
__global__ __launch_bounds__(kThreads) void single_proj_f32(SingleAttnF32Args p) {
  __shared__ float xn[kRows][kMaxCs];
  const long rows = (long)p.B * p.N, pos0 = (long)blockIdx.x * kRows;
  const int C = p.C, HD = p.H * p.D;
  norm_rows(p.a, pos0, rows, C, p.ln_w, p.ln_b, xn);
  __syncthreads();
  const float scale = 1.0f / sqrtf((float)p.D);
  for (int idx = threadIdx.x; idx < kRows * 4 * HD; idx += kThreads) {
    const int r = idx / (4 * HD), o = idx % (4 * HD), kind = o / HD, ch = o % HD;
    if (pos0 + r >= rows) continue;
    const float* W = kind == 0 ? p.wq : kind == 1 ? p.wk : kind == 2 ? p.wv : p.wg;
    float v = dot_f32(xn[r], W + (size_t)ch * C, C);
    if (kind == 0) v = (v + p.bq[ch]) * scale;
    if (kind == 3) v = sigmoid_f32(v);
    float* dst = kind == 0 ? p.q : kind == 1 ? p.k : kind == 2 ? p.v : p.g;
    dst[(pos0 + r) * HD + ch] = v;
  }
}

// one thread per query of one (batch, head); keys in chunks of 32 through LDS together with the
// [128 queries][32 keys] slice of the pair bias; online softmax; output times gate
template <int DMAX>
__global__ __launch_bounds__(128) void single_attn_f32(SingleAttnF32Args p) {
  constexpr int KC = 32;
  __shared__ float ks[KC][DMAX], vs[KC][DMAX], mbs[KC];
  __shared__ float pbs[128][KC + 1];
  const int N = p.N, H = p.H, D = p.D, HD = H * D;
  const int qg = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  const int qi = qg * 128 + threadIdx.x;
  const bool active = qi < N;
  float qv[DMAX], ov[DMAX];
#pragma unroll
  for (int d = 0; d < DMAX; ++d) {
    qv[d] = (active && d < D) ? p.q[((size_t)b * N + qi) * HD + h * D + d] : 0.f;
    ov[d] = 0.f;
  }
  const float* pb = p.pair_bias + (((size_t)b * H + h) * N + (size_t)qg * 128) * N;
  float m = -__builtin_inff(), l = 0.f;
  for (int k0 = 0; k0 < N; k0 += KC) {
    __syncthreads();
    for (int e = threadIdx.x; e < KC * DMAX; e += 128) {
      const int kk = e / DMAX, d = e % DMAX;
      const bool in = k0 + kk < N && d < D;
      ks[kk][d] = in ? p.k[((size_t)b * N + k0 + kk) * HD + h * D + d] : 0.f;
      vs[kk][d] = in ? p.v[((size_t)b * N + k0 + kk) * HD + h * D + d] : 0.f;
    }
    for (int e = threadIdx.x; e < 128 * KC; e += 128) {
      const int r = e / KC, c = e % KC;
      pbs[r][c] = (qg * 128 + r < N && k0 + c < N) ? pb[(size_t)r * N + k0 + c] : 0.f;
    }
    if (threadIdx.x < KC) {
      const int kx = k0 + threadIdx.x;
      float mv = 1.f;
      if (kx < N && p.mask) mv = p.mask[(size_t)b * N + kx];
      mbs[threadIdx.x] = p.inf * (mv - 1.f);
    }
    __syncthreads();
    const int kn = N - k0 < KC ? N - k0 : KC;
    float s[KC];
    float cmax = -__builtin_inff();
#pragma unroll
    for (int kk = 0; kk < KC; ++kk) {
      float acc = 0.f;
#pragma unroll
      for (int d = 0; d < DMAX; ++d) acc = fmaf(qv[d], ks[kk][d], acc);
      // logits in the reference's order: q.k, then the mask bias, then the pair bias
      acc = acc + mbs[kk];
      acc = acc + pbs[threadIdx.x][kk];
      s[kk] = kk < kn ? acc : -__builtin_inff();
      cmax = fmaxf(cmax, s[kk]);
    }
    const float m_new = fmaxf(m, cmax);
    const float alpha = expf(m - m_new);
    l *= alpha;
#pragma unroll
    for (int d = 0; d < DMAX; ++d) ov[d] *= alpha;
#pragma unroll
    for (int kk = 0; kk < KC; ++kk) {
      const float pw = expf(s[kk] - m_new);
      l += pw;
#pragma unroll
      for (int d = 0; d < DMAX; ++d) ov[d] = fmaf(pw, vs[kk][d], ov[d]);
    }
    m = m_new;
  }
  if (active) {
    const float inv = 1.0f / l;
    const size_t off = ((size_t)b * N + qi) * HD + h * D;
#pragma unroll
    for (int d = 0; d < DMAX; ++d)
      if (d < D) p.og[off + d] = (ov[d] * inv) * p.g[off + d];
  }
}

__global__ __launch_bounds__(kThreads) void single_out_f32(SingleAttnF32Args p) {
  __shared__ float og[kRows][kMaxCs];
  const long rows = (long)p.B * p.N, pos0 = (long)blockIdx.x * kRows;
  const int C = p.C, HD = p.H * p.D;
  for (int idx = threadIdx.x; idx < kRows * HD; idx += kThreads) {
    const int r = idx / HD, c = idx % HD;
    og[r][c] = pos0 + r < rows ? p.og[(pos0 + r) * HD + c] : 0.f;
  }
  __syncthreads();
  for (int idx = threadIdx.x; idx < kRows * C; idx += kThreads) {
    const int r = idx / C, o = idx % C;
    if (pos0 + r >= rows) continue;
    float v = dot_f32(og[r], p.wo + (size_t)o * HD, HD);
    if (p.add_residual) v = p.a[(pos0 + r) * C + o] + v;
    p.out[(pos0 + r) * C + o] = v;
  }
}

// out = [x +] ((silu(LN(x) Wa^T) * (LN(x) Wb^T)) Wout^T) * mask for kRows rows per work-group; the
// hidden activations stay in LDS
__global__ __launch_bounds__(kThreads) void row_transition_f32(RowTransitionF32Args p) {
  __shared__ float xn[kRows][kMaxCs];
  __shared__ float hid[kRows][kMaxHidden];
  const long pos0 = (long)blockIdx.x * kRows;
  const int C = p.C, HID = p.HID;
  norm_rows(p.x, pos0, p.rows, C, p.ln_w, p.ln_b, xn);
  __syncthreads();
  for (int idx = threadIdx.x; idx < kRows * HID; idx += kThreads) {
    const int r = idx / HID, o = idx % HID;
    const float a = dot_f32(xn[r], p.wa + (size_t)o * C, C);
    const float b = dot_f32(xn[r], p.wb + (size_t)o * C, C);
    hid[r][o] = (a * sigmoid_f32(a)) * b;  // silu(a) * b (activations.py:60-61)
  }
  __syncthreads();
  for (int idx = threadIdx.x; idx < kRows * C; idx += kThreads) {
    const int r = idx / C, o = idx % C;
    if (pos0 + r >= p.rows) continue;
    float v = dot_f32(hid[r], p.wout + (size_t)o * HID, HID);
    if (p.mask) v = v * p.mask[pos0 + r];
    if (p.add_residual) v = p.x[(pos0 + r) * C + o] + v;
    p.out[(pos0 + r) * C + o] = v;
  }
}

}  // namespace

hipError_t single_attn_fwd_f32(const SingleAttnF32Args& a, hipStream_t stream) {
  if (a.C < 1 || a.C > kMaxCs || a.H < 1 || a.D < 1 || a.D > 64 || a.H * a.D > kMaxCs || a.N < 1 || a.B < 1 ||
      a.B > 65535 || a.H > 65535)
    return hipErrorInvalidValue;
  const long rows = (long)a.B * a.N;
  const long blocks = (rows + kRows - 1) / kRows;
  if (blocks > 0x7fffffffl) return hipErrorInvalidValue;
  hipLaunchKernelGGL(single_proj_f32, dim3((unsigned)blocks), dim3(kThreads), 0, stream, a);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return e;
  const dim3 grid((a.N + 127) / 128, a.H, a.B);
  if (a.D <= 32) hipLaunchKernelGGL(single_attn_f32<32>, grid, dim3(128), 0, stream, a);
  else hipLaunchKernelGGL(single_attn_f32<64>, grid, dim3(128), 0, stream, a);
  e = hipGetLastError();
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(single_out_f32, dim3((unsigned)blocks), dim3(kThreads), 0, stream, a);
  return hipGetLastError();
}

hipError_t row_transition_fwd_f32(const RowTransitionF32Args& a, hipStream_t stream) {
  if (a.rows < 1 || a.C < 1 || a.C > kMaxCs || a.HID < 1 || a.HID > kMaxHidden) return hipErrorInvalidValue;
  const long blocks = (a.rows + kRows - 1) / kRows;
  if (blocks > 0x7fffffffl) return hipErrorInvalidValue;
  hipLaunchKernelGGL(row_transition_f32, dim3((unsigned)blocks), dim3(kThreads), 0, stream, a);
  return hipGetLastError();
}

}  // namespace of3

// fp32 path of the two pair-stack updates (OF3_DTYPE_F32): the reference's default inference
// precision (fp32 end to end).  Same mathematics and the same rounding-free order of
// operations as the reference's stock PyTorch path:
//   triangle multiplication   triangular_multiplicative_update.py:482-503, :71-97
//   triangle attention        triangular_attention.py:102-167, attention.py:94-135,265-302
//   pair transition           transition.py:225-271, activations.py:33-61
//   pair-bias projection      attention_pair_bias.py:151-161
// These kernels are written for exactness and generality (any N, C, C_hidden <= 256, head
// width <= 64) with full-precision expf in the gates (the softmax uses the hardware exp2); they are the precision reference of the library on the
// GPU, not its fast path (that is the bf16 path).  The linear layers of the position-wise passes
// run on the fp32 matrix pipe (v_mfma_f32_32x32x2_f32: exact fp32 products, fp32 sums) in
// work-groups of 32 positions whenever the channel counts are multiples of 8 and the weights are
// 16-byte aligned; plain FMA kernels of 8 positions serve every other shape.
//
// Layouts (workspace, fp32): a, b, x  [B][CH][N][N] with a[b][c][i][k] (k contracted);
// q, k, v [B][N(i)][H][N(j)][D]; triangle bias [B][H][N][N]; o [B][N][N][H*D].
#include <cstdint>
#include <initializer_list>

#include "of3_device.h"
#include "of3_kernels.h"
#include "of3_launch.h"

namespace of3 {

namespace {

constexpr int kP = 8;        // positions per work-group in the position-wise kernels
constexpr int kThreads = 256;
constexpr int kMaxC = 256;
constexpr float kEps = 1e-5f;

constexpr float kLog2eF32 = 1.4426950408889634f;
__device__ __forceinline__ float sigmoid_f32(float x) { return 1.0f / (1.0f + expf(-x)); }
// the matrix-pipe kernels: the hardware's exp2 and reciprocal (1 ulp each; the rounding of x * log2(e)
// adds |x| * 2^-24 relative), a sixth of the instructions
__device__ __forceinline__ float sigmoid_hw_f32(float x) {
  return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-x * kLog2eF32));
}

// LayerNorm of kP positions (32 lanes each) from global rows into shared xn[kP][C].
// src(pos) returns the pointer to the C channels of position pos or nullptr (out of range).
template <typename Src>
__device__ __forceinline__ void layer_norm_rows(Src src, const float* __restrict__ w, const float* __restrict__ bsh,
                                                int C, float (*xn)[kMaxC]) {
  const int pos = threadIdx.x >> 5, l = threadIdx.x & 31;
  const float* row = src(pos);
  float s = 0.f;
  if (row)
    for (int c = l; c < C; c += 32) s += row[c];
#pragma unroll
  for (int o = 16; o > 0; o >>= 1) s += __shfl_xor(s, o, 32);
  const float mean = s / (float)C;
  float q = 0.f;
  if (row)
    for (int c = l; c < C; c += 32) {
      const float d = row[c] - mean;
      q += d * d;
    }
#pragma unroll
  for (int o = 16; o > 0; o >>= 1) q += __shfl_xor(q, o, 32);
  const float rstd = 1.0f / sqrtf(q / (float)C + kEps);
  for (int c = l; c < C; c += 32) xn[pos][c] = row ? (row[c] - mean) * rstd * w[c] + bsh[c] : 0.f;
}

__device__ __forceinline__ float dot_row(const float* __restrict__ x, const float* __restrict__ w, int n) {
  float acc = 0.f;
  for (int k = 0; k < n; ++k) acc = fmaf(x[k], w[k], acc);
  return acc;
}


// ---- linear layers on the fp32 matrix pipe ---------------------------------------------------
constexpr int kTP = 32;  // positions per work-group of the matrix-pipe kernels

// row of accumulator register v in lane half lh of a 32 x 32 MFMA result (the lane's column is lane & 31)
__device__ __forceinline__ int acc_row(int v, int lh) { return 8 * (v >> 2) + 4 * lh + (v & 3); }

// LayerNorm of kTP positions (32 lanes each) into the LDS tile xn[kTP][ldx]; same arithmetic as
// layer_norm_rows
template <typename Src>
__device__ __forceinline__ void layer_norm_tile(Src src, const float* __restrict__ w, const float* __restrict__ bsh,
                                                int C, float* xn, int ldx) {
  const int l = threadIdx.x & 31;
  for (int pos = threadIdx.x >> 5; pos < kTP; pos += kThreads / 32) {
    const float* row = src(pos);
    float s = 0.f;
    if (row)
      for (int c = l; c < C; c += 32) s += row[c];
#pragma unroll
    for (int o = 16; o > 0; o >>= 1) s += __shfl_xor(s, o, 32);
    const float mean = s / (float)C;
    float q = 0.f;
    if (row)
      for (int c = l; c < C; c += 32) {
        const float d = row[c] - mean;
        q += d * d;
      }
#pragma unroll
    for (int o = 16; o > 0; o >>= 1) q += __shfl_xor(q, o, 32);
    const float rstd = 1.0f / sqrtf(q / (float)C + kEps);
    for (int c = l; c < C; c += 32) xn[pos * ldx + c] = row ? (row[c] - mean) * rstd * w[c] + bsh[c] : 0.f;
  }
}

// NW linear layers at once for one 32 x 32 tile: the kTP positions of the LDS tile xs[kTP][ldx]
// (K values per row, K % 8 == 0, 16-byte aligned rows) against rows o0 .. o0+31 of each W[n]
// ([n_out][K] row-major, 16-byte aligned; rows past n_out-1 repeat the last one and are not
// used by the caller).  The summation index is dealt so that both operands are read as float4:
// MFMA step 4j+e pairs k = 8j+e (lanes 0-31) with k = 8j+4+e (lanes 32-63).
// OUT_ROWS: the outputs are the MFMA rows (lane & 31 = position, register v = output
// o0 + acc_row(v, lh)); otherwise the positions are (lane & 31 = output o0 + ..., register v =
// position acc_row(v, lh)).  The caller picks whichever makes its stores contiguous over lanes.
// ldw: row stride of W (K when the whole row is summed; larger when xs holds a slice of the inputs
// and W points at that slice's first column); ACCUMULATE keeps the values acc came in with.
template <int NW, bool OUT_ROWS, bool ACCUMULATE = false>
__device__ __forceinline__ void linear_tiles(const float* xs, int ldx, const float* const (&W)[NW], int o0, int n_out,
                                             int K, f32x16_t (&acc)[NW], int ldw = 0) {
  if (ldw == 0) ldw = K;
  const int lane = threadIdx.x & 63, l32 = lane & 31, lh = lane >> 5;
  int row = o0 + l32;
  row = row < n_out ? row : n_out - 1;
  const float4* xr = reinterpret_cast<const float4*>(xs + l32 * ldx + 4 * lh);
  const float4* wr[NW];
#pragma unroll
  for (int n = 0; n < NW; ++n) {
    wr[n] = reinterpret_cast<const float4*>(W[n] + (size_t)row * ldw + 4 * lh);
    if (!ACCUMULATE) acc[n] = zero16();
  }
  const int steps = K / 8;
  for (int j = 0; j < steps; ++j) {
    const float4 x = xr[2 * j];
#pragma unroll
    for (int n = 0; n < NW; ++n) {
      const float4 w = wr[n][2 * j];
      if (OUT_ROWS) {
        acc[n] = __builtin_amdgcn_mfma_f32_32x32x2f32(w.x, x.x, acc[n], 0, 0, 0);
        acc[n] = __builtin_amdgcn_mfma_f32_32x32x2f32(w.y, x.y, acc[n], 0, 0, 0);
        acc[n] = __builtin_amdgcn_mfma_f32_32x32x2f32(w.z, x.z, acc[n], 0, 0, 0);
        acc[n] = __builtin_amdgcn_mfma_f32_32x32x2f32(w.w, x.w, acc[n], 0, 0, 0);
      } else {
        acc[n] = __builtin_amdgcn_mfma_f32_32x32x2f32(x.x, w.x, acc[n], 0, 0, 0);
        acc[n] = __builtin_amdgcn_mfma_f32_32x32x2f32(x.y, w.y, acc[n], 0, 0, 0);
        acc[n] = __builtin_amdgcn_mfma_f32_32x32x2f32(x.z, w.z, acc[n], 0, 0, 0);
        acc[n] = __builtin_amdgcn_mfma_f32_32x32x2f32(x.w, w.w, acc[n], 0, 0, 0);
      }
    }
  }
}


// ---- linear layers with fp32 operands split into three bf16 terms -------------------------------
// x = xh + xm + xl with xh = bf16(x), xm = bf16(x - xh), xl = bf16(x - xh - xm): both differences are
// exact in fp32, so the three terms carry 24 significant bits of x.  A product then is
//     x w = xh wh + xh wm + xm wh + xh wl + xl wh + xm wm + (three terms below 2^-24 |x w|),
// six bf16 MFMA products (exact, summed in fp32) at a sixteenth of the cost of an fp32 MFMA product each:
// 2.7 times less matrix time for the accuracy of an fp32 product.  The activations are split once per
// tile when the LayerNorm writes them to LDS; the weights once per call into the workspace, in the
// order the MFMA A/B operands are read: the 16 bytes lane l needs for step s of row tile t sit at
// ((t * steps + s) * 64 + l) * 16, so a wave's operand read is one contiguous kilobyte (read straight
// from the row-major matrix the same operand touches 32 cache lines, and the passes are bound by that).
struct Split3 {
  bf16_t h, m, l;
};
__device__ __forceinline__ Split3 split3(float v) {
  Split3 s;
  s.h = to_bf16(v);
  const float r1 = v - bf16_to_f32(s.h);
  s.m = to_bf16(r1);
  s.l = to_bf16(r1 - bf16_to_f32(s.m));
  return s;
}

// eight values at once, as three MFMA operands of 8 bf16
__device__ __forceinline__ void split8(const float (&x)[8], u32x4_t& h, u32x4_t& m, u32x4_t& l) {
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    const float a = x[2 * w], b = x[2 * w + 1];
    const uint32_t ph = pack_bf16(a, b);
    const float ra = a - __uint_as_float(ph << 16), rb = b - __uint_as_float(ph & 0xffff0000u);
    const uint32_t pm = pack_bf16(ra, rb);
    const float sa = ra - __uint_as_float(pm << 16), sb = rb - __uint_as_float(pm & 0xffff0000u);
    h[w] = ph;
    m[w] = pm;
    l[w] = pack_bf16(sa, sb);
  }
}

// LDS tile of tp positions in three planes [tp][ld] bf16 (ld = K + 8: rows 16 bytes apart in the bank map)
struct TileX3 {
  bf16_t* h;
  int ld, plane;  // plane = tp * ld elements: m = h + plane, l = h + 2 * plane
  __device__ __forceinline__ void store(int pos, int c, float v) const {
    const Split3 s = split3(v);
    h[pos * ld + c] = s.h;
    h[plane + pos * ld + c] = s.m;
    h[2 * plane + pos * ld + c] = s.l;
  }
  // the same tile from position `rows` on
  __device__ __forceinline__ TileX3 at(int rows) const {
    TileX3 t = *this;
    t.h += rows * ld;
    return t;
  }
  // two adjacent channels c (even) and c + 1 in one 4-byte write per plane
  __device__ __forceinline__ void store2(int pos, int c, float v0, float v1) const {
    const uint32_t ph = pack_bf16(v0, v1);
    const float r0 = v0 - __uint_as_float(ph << 16), r1 = v1 - __uint_as_float(ph & 0xffff0000u);
    const uint32_t pm = pack_bf16(r0, r1);
    const float s0 = r0 - __uint_as_float(pm << 16), s1 = r1 - __uint_as_float(pm & 0xffff0000u);
    uint32_t* d = reinterpret_cast<uint32_t*>(h + pos * ld + c);
    d[0] = ph;
    d[plane / 2] = pm;
    d[plane] = pack_bf16(s0, s1);
  }
};
__device__ __forceinline__ TileX3 make_tile_x3(void* base, int K, int tp) {
  TileX3 t;
  t.h = static_cast<bf16_t*>(base);
  t.ld = K + 8;
  t.plane = tp * t.ld;
  return t;
}
__host__ __device__ constexpr size_t tile_bytes_x3(int K, int tp) { return (size_t)3 * tp * (K + 8) * sizeof(bf16_t); }

// split, operand-ordered copy of a weight matrix [rows][K]: three planes of ceil(rows / 32) * 32 * K bf16
struct WeightX3 {
  const bf16_t* h;
  long plane;
};
__host__ __device__ constexpr long packed_elems(long rows, long K) { return (rows + 31) / 32 * 32 * K; }

// up to six matrices in one launch
struct SplitJobs {
  static constexpr int kMax = 6;
  const float* src[kMax];
  bf16_t* dst[kMax];
  int rows[kMax], K[kMax];
  long first[kMax + 1];  // first item of each matrix; first[n] = all items
  int n;
};

__global__ __launch_bounds__(kThreads) void split_weights_f32(SplitJobs j) {
  // one thread per (matrix, row tile, step, lane): its 8 consecutive k-values
  const long gitem = (long)blockIdx.x * kThreads + threadIdx.x;
  if (gitem >= j.first[j.n]) return;
  int q = 0;
#pragma unroll
  for (int i = 1; i < SplitJobs::kMax; ++i)
    if (i < j.n && gitem >= j.first[i]) q = i;
  const float* __restrict__ src = j.src[q];
  bf16_t* __restrict__ dst = j.dst[q];
  const int rows = j.rows[q], K = j.K[q];
  const long item = gitem - j.first[q];
  const int steps = K / 16;
  const int lane = (int)(item & 63), l32 = lane & 31, lh = lane >> 5;
  const long ts = item >> 6;
  const int s = (int)(ts % steps), t = (int)(ts / steps);
  int row = 32 * t + l32;
  row = row < rows ? row : rows - 1;  // rows past the end repeat the last one (their results are dropped)
  const long plane = packed_elems(rows, K);
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const Split3 v = split3(src[(size_t)row * K + 16 * s + 8 * lh + e]);
    dst[item * 8 + e] = v.h;
    dst[plane + item * 8 + e] = v.m;
    dst[2 * plane + item * 8 + e] = v.l;
  }
}

// host side: matrices are added one after the other into the workspace, then split by one launch
struct WeightSplitter {
  SplitJobs j;
  bf16_t* w;
  explicit WeightSplitter(void* workspace) : j(), w(static_cast<bf16_t*>(workspace)) {}
  void add(const float* src, int rows, int K, WeightX3& dst) {
    dst.h = w;
    dst.plane = packed_elems(rows, K);
    j.src[j.n] = src;
    j.dst[j.n] = w;
    j.rows[j.n] = rows;
    j.K[j.n] = K;
    j.first[j.n + 1] = j.first[j.n] + dst.plane / 8;
    ++j.n;
    w += 3 * dst.plane;
  }
  hipError_t launch(hipStream_t stream) const {
    const long items = j.first[j.n];
    hipLaunchKernelGGL(split_weights_f32, dim3((unsigned)((items + kThreads - 1) / kThreads)), dim3(kThreads), 0, stream, j);
    return hipGetLastError();
  }
};

// LayerNorm of 32 * TILES positions by NT threads into a split tile, a row per 32 lanes, at most 256 channels (a
// multiple of 16).  Lane l holds channels 2 l + 64 e and 2 l + 64 e + 1, e < 4.  A row is read once
// and kept in registers (the reads of four rows are in flight together).  extra(pos, y) sees the
// normalised row: y[2 e + i] is channel 2 l + 64 e + i.
// FAST: the channel count is a multiple of 64 (whole wave-uniform steps instead of lane masks) and
// the rows are 8-byte aligned (one read per pair).
//
// The work comes in two halves, so that a persistent work-group can have the rows of its next tile
// in flight while it multiplies the current one: ln_rows_load issues the reads (src(pos, valid)
// returns an address that can always be read, of a real row, and says whether the position exists:
// no read is under a lane condition, which would make the compiler wait for every read in flight),
// ln_rows_store normalises, splits and writes the tile.
template <int TILES, int NT>
struct LnRows {
  static constexpr int kGroups = NT / 32, ITERS = 32 * TILES / kGroups;
  float val[ITERS][8];
  bool has[ITERS];
};

template <int TILES, bool FAST, int NT, typename Src>
__device__ __forceinline__ void ln_rows_load(Src src, int C, LnRows<TILES, NT>& r) {
  constexpr int kGroups = NT / 32, ITERS = LnRows<TILES, NT>::ITERS;
  const int l = threadIdx.x & 31, grp = threadIdx.x >> 5;
  const int nE = C / 64;
#pragma unroll
  for (int u = 0; u < ITERS; ++u) {
    bool valid;
    const float* row = src(grp + u * kGroups, valid);
    r.has[u] = valid;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      if (FAST) {
        if (e < nE) {
          const float2 v = *reinterpret_cast<const float2*>(row + 2 * l + 64 * e);
          r.val[u][2 * e] = v.x, r.val[u][2 * e + 1] = v.y;
        } else {
          r.val[u][2 * e] = r.val[u][2 * e + 1] = 0.f;
        }
      } else {
        const bool in = 2 * l + 64 * e < C;
        r.val[u][2 * e] = in ? row[2 * l + 64 * e] : 0.f;
        r.val[u][2 * e + 1] = in ? row[2 * l + 64 * e + 1] : 0.f;
      }
    }
  }
}

template <int TILES, bool FAST, int NT, typename Extra>
__device__ __forceinline__ void ln_rows_store(const LnRows<TILES, NT>& r, const float* __restrict__ w,
                                              const float* __restrict__ bsh, int C, const TileX3& t, Extra extra) {
  constexpr int kGroups = NT / 32, ITERS = LnRows<TILES, NT>::ITERS;
  const int l = threadIdx.x & 31, grp = threadIdx.x >> 5;
  const int nE = C / 64;
  auto ok = [&](int e) { return FAST ? e < nE : 2 * l + 64 * e < C; };
  float wv[8], bv[8];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const int c = 2 * l + 64 * e;
    wv[2 * e] = wv[2 * e + 1] = bv[2 * e] = bv[2 * e + 1] = 0.f;
    if (ok(e)) {
      wv[2 * e] = w[c], wv[2 * e + 1] = w[c + 1];
      bv[2 * e] = bsh[c], bv[2 * e + 1] = bsh[c + 1];
    }
  }
#pragma unroll
  for (int u = 0; u < ITERS; ++u) {
    const int pos = grp + u * kGroups;
    float s = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) s += r.val[u][e];  // channels past C hold 0
#pragma unroll
    for (int o = 16; o > 0; o >>= 1) s += __shfl_xor(s, o, 32);
    const float mean = s / (float)C;
    float q = 0.f;
#pragma unroll
    for (int e = 0; e < 4; ++e)
      if (ok(e)) {
        const float d0 = r.val[u][2 * e] - mean, d1 = r.val[u][2 * e + 1] - mean;
        q += d0 * d0;
        q += d1 * d1;
      }
#pragma unroll
    for (int o = 16; o > 0; o >>= 1) q += __shfl_xor(q, o, 32);
    const float rstd = 1.0f / sqrtf(q / (float)C + kEps);
    float y[8];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      y[2 * e] = r.has[u] ? (r.val[u][2 * e] - mean) * rstd * wv[2 * e] + bv[2 * e] : 0.f;
      y[2 * e + 1] = r.has[u] ? (r.val[u][2 * e + 1] - mean) * rstd * wv[2 * e + 1] + bv[2 * e + 1] : 0.f;
      if (ok(e)) t.store2(pos, 2 * l + 64 * e, y[2 * e], y[2 * e + 1]);
    }
    extra(pos, y);
  }
}

template <int TILES, bool FAST, int NT, typename Src, typename Extra>
__device__ __forceinline__ void layer_norm_tile_x3(Src src, const float* __restrict__ w, const float* __restrict__ bsh,
                                                   int C, const TileX3& t, Extra extra) {
  LnRows<TILES, NT> r;
  ln_rows_load<TILES, FAST, NT>(src, C, r);
  ln_rows_store<TILES, FAST, NT>(r, w, bsh, C, t, extra);
}
struct NoExtra {
  __device__ __forceinline__ void operator()(int, const float (&)[8]) const {}
};

// linear_tiles on split operands for XT tiles of 32 positions at once (a weight operand is read once
// for all of them): K % 16 == 0, o0 a multiple of 32; lane (row or column l32, half lh) supplies the 8
// consecutive k-values 16 s + 8 lh .. + 7 of step s, one 16-byte read per term and operand.  The
// result layout of acc[n][xt] is that of linear_tiles for positions 32 xt .. 32 xt + 31.
// ACCUMULATE: acc is added to.  A slice of a wider weight matrix: w_step0 = its first k-step,
// w_steps = the matrix's k-steps per row tile (0: K / 16, the whole width).
template <int NW, int XT, bool OUT_ROWS, bool ACCUMULATE = false>
__device__ __forceinline__ void linear_tiles_x3(const TileX3& xs, const WeightX3 (&W)[NW], int o0, int K,
                                                f32x16_t (&acc)[NW][XT], int w_step0 = 0, int w_steps = 0) {
  const int lane = threadIdx.x & 63, l32 = lane & 31, lh = lane >> 5;
  const int steps = K / 16;
  if (w_steps == 0) w_steps = steps;
  const u32x4_t* xh = reinterpret_cast<const u32x4_t*>(xs.h + l32 * xs.ld + 8 * lh);
  const int xplane = xs.plane / 8, xtile = 32 * xs.ld / 8;  // in 16-byte units
  const u32x4_t* wh[NW];
  long wplane[NW];
#pragma unroll
  for (int n = 0; n < NW; ++n) {
    wh[n] = reinterpret_cast<const u32x4_t*>(W[n].h) + ((size_t)(o0 >> 5) * w_steps + w_step0) * 64 + lane;
    wplane[n] = W[n].plane / 8;
    if (!ACCUMULATE) {
#pragma unroll
      for (int xt = 0; xt < XT; ++xt) acc[n][xt] = zero16();
    }
  }
  for (int s = 0; s < steps; ++s) {
    u32x4_t x_h[XT], x_m[XT], x_l[XT];
#pragma unroll
    for (int xt = 0; xt < XT; ++xt) {
      x_h[xt] = xh[xt * xtile + 2 * s];
      x_m[xt] = xh[xplane + xt * xtile + 2 * s];
      x_l[xt] = xh[2 * xplane + xt * xtile + 2 * s];
    }
#pragma unroll
    for (int n = 0; n < NW; ++n) {
      const u32x4_t w_h = wh[n][64 * s], w_m = wh[n][wplane[n] + 64 * s], w_l = wh[n][2 * wplane[n] + 64 * s];
#pragma unroll
      for (int xt = 0; xt < XT; ++xt) {
        // smallest terms first
        if (OUT_ROWS) {
          acc[n][xt] = mfma_32x32x16(w_l, x_h[xt], acc[n][xt]);
          acc[n][xt] = mfma_32x32x16(w_h, x_l[xt], acc[n][xt]);
          acc[n][xt] = mfma_32x32x16(w_m, x_m[xt], acc[n][xt]);
          acc[n][xt] = mfma_32x32x16(w_m, x_h[xt], acc[n][xt]);
          acc[n][xt] = mfma_32x32x16(w_h, x_m[xt], acc[n][xt]);
          acc[n][xt] = mfma_32x32x16(w_h, x_h[xt], acc[n][xt]);
        } else {
          acc[n][xt] = mfma_32x32x16(x_h[xt], w_l, acc[n][xt]);
          acc[n][xt] = mfma_32x32x16(x_l[xt], w_h, acc[n][xt]);
          acc[n][xt] = mfma_32x32x16(x_m[xt], w_m, acc[n][xt]);
          acc[n][xt] = mfma_32x32x16(x_h[xt], w_m, acc[n][xt]);
          acc[n][xt] = mfma_32x32x16(x_m[xt], w_h, acc[n][xt]);
          acc[n][xt] = mfma_32x32x16(x_h[xt], w_h, acc[n][xt]);
        }
      }
    }
  }
}

// ---- triangle multiplication -----------------------------------------------------------------
struct TrimulF32 {
  const float *z, *mask;
  PairView zv, mv;          // view used by the projection pass (swapped for the incoming update)
  PairView zc;              // canonical view (output pass)
  const float *ln_in_w, *ln_in_b, *ln_out_w, *ln_out_b;
  const float *w_ap, *w_ag, *w_bp, *w_bg, *w_g, *w_z;
  WeightX3 s_ap, s_ag, s_bp, s_bg, s_g, s_z;  // split copies (the *_x3 kernels only)
  float *a, *b, *x, *out;
  // a and b split into three bf16 terms in the k-panel layout (the split-operand contraction only):
  // element (b, c, r, k) of a term sits at ((((b CH + c) Np / 32 + k / 32) Np + r) 32 + k % 32, the
  // three terms ab_plane elements apart; Np = N rounded up to whole 32-wide panels
  bf16_t *as, *bs;
  long ab_plane;
  int Np;
  int B, N, C, CH, add_residual;
};

__global__ __launch_bounds__(kThreads) void trimul_proj_f32(TrimulF32 p, int groups) {
  __shared__ float xn[kP][kMaxC];
  __shared__ float msk[kP];
  const int N = p.N, C = p.C, CH = p.CH;
  const int g = blockIdx.x % groups, r = (blockIdx.x / groups) % N, b = blockIdx.x / (groups * N);
  const int k0 = g * kP;
  layer_norm_rows(
      [&](int pos) -> const float* {
        const int k = k0 + pos;
        return k < N ? p.z + b * p.zv.stride_b + r * p.zv.stride_r + k * p.zv.stride_k : nullptr;
      },
      p.ln_in_w, p.ln_in_b, C, xn);
  if (threadIdx.x < kP) {
    const int k = k0 + threadIdx.x;
    msk[threadIdx.x] = (k < N && p.mask) ? p.mask[b * p.mv.stride_b + r * p.mv.stride_r + k * p.mv.stride_k] : 1.f;
  }
  __syncthreads();
  for (int idx = threadIdx.x; idx < kP * CH; idx += kThreads) {
    const int pos = idx % kP, c = idx / kP, k = k0 + pos;
    if (k >= N) continue;
    const float m = msk[pos];
    // a = mask * sigmoid(gate) * projection, in the reference's order of multiplication
    const float av = m * sigmoid_f32(dot_row(xn[pos], p.w_ag + c * C, C)) * dot_row(xn[pos], p.w_ap + c * C, C);
    const float bv = m * sigmoid_f32(dot_row(xn[pos], p.w_bg + c * C, C)) * dot_row(xn[pos], p.w_bp + c * C, C);
    const size_t o = (((size_t)b * CH + c) * N + r) * N + k;
    p.a[o] = av;
    p.b[o] = bv;
  }
}

// x[p][i][j] = sum_k a[p][i][k] * b[p][j][k]: 64 x 64 tile, 4 x 4 outputs per thread
__global__ __launch_bounds__(kThreads) void trimul_contract_f32(const float* __restrict__ a, const float* __restrict__ b,
                                                               float* __restrict__ x, int N) {
  constexpr int T = 64, BK = 16;
  __shared__ float as[BK][T + 4], bs[BK][T + 4];
  const size_t plane = (size_t)blockIdx.z * N * N;
  const int i0 = blockIdx.y * T, j0 = blockIdx.x * T;
  const int ty = threadIdx.x / 16, tx = threadIdx.x % 16;
  float acc[4][4] = {};
  for (int k0 = 0; k0 < N; k0 += BK) {
    for (int e = threadIdx.x; e < T * BK; e += kThreads) {
      const int row = e / BK, kk = e % BK;
      const bool kin = k0 + kk < N;
      as[kk][row] = (kin && i0 + row < N) ? a[plane + (size_t)(i0 + row) * N + k0 + kk] : 0.f;
      bs[kk][row] = (kin && j0 + row < N) ? b[plane + (size_t)(j0 + row) * N + k0 + kk] : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < BK; ++kk) {
      float av[4], bv[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        av[u] = as[kk][ty * 4 + u];
        bv[u] = bs[kk][tx * 4 + u];
      }
#pragma unroll
      for (int u = 0; u < 4; ++u)
#pragma unroll
        for (int v = 0; v < 4; ++v) acc[u][v] = fmaf(av[u], bv[v], acc[u][v]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int u = 0; u < 4; ++u)
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const int i = i0 + ty * 4 + u, j = j0 + tx * 4 + v;
      if (i < N && j < N) x[plane + (size_t)i * N + j] = acc[u][v];
    }
}

// the same on the fp32 matrix pipe: 128 x 128 tile, four waves of 64 x 64 (2 x 2 MFMA blocks).
// a and b chunks of 32 k-values sit in LDS as [row][32 + 4] so that a lane's operand values for four
// MFMA steps are one float4 (step 4j+e pairs k = 8j+e in lanes 0-31 with k = 8j+4+e in lanes 32-63);
// i is the MFMA row side and j the column side: the lanes of a store cover 32 consecutive j.
__global__ __launch_bounds__(kThreads) void trimul_contract_mm_f32(const float* __restrict__ a,
                                                                  const float* __restrict__ b,
                                                                  float* __restrict__ x, int N) {
  constexpr int T = 128, BK = 32, LD = BK + 4;
  __shared__ __align__(16) float as[T * LD];
  __shared__ __align__(16) float bs[T * LD];
  const size_t plane = (size_t)blockIdx.z * N * N;
  const int i0 = blockIdx.y * T, j0 = blockIdx.x * T;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, l32 = lane & 31, lh = lane >> 5;
  const int wi = 64 * (wave >> 1), wj = 64 * (wave & 1);
  f32x16_t acc[2][2];
#pragma unroll
  for (int u = 0; u < 2; ++u)
#pragma unroll
    for (int v = 0; v < 2; ++v) acc[u][v] = zero16();
  // a chunk travels global -> registers while the previous one is multiplied, and registers -> LDS
  // between two barriers; a wave's load covers two rows of 128 contiguous bytes
  constexpr int LI = T * BK / kThreads;
  float a_r[LI], b_r[LI];
  const int ld_row = threadIdx.x / BK, ld_k = threadIdx.x % BK;  // + it * (kThreads / BK) rows
  auto fetch = [&](int k0) {
    const bool kin = k0 + ld_k < N;
#pragma unroll
    for (int it = 0; it < LI; ++it) {
      const int row = ld_row + it * (kThreads / BK);
      a_r[it] = (kin && i0 + row < N) ? a[plane + (size_t)(i0 + row) * N + k0 + ld_k] : 0.f;
      b_r[it] = (kin && j0 + row < N) ? b[plane + (size_t)(j0 + row) * N + k0 + ld_k] : 0.f;
    }
  };
  fetch(0);
  for (int k0 = 0; k0 < N; k0 += BK) {
    __syncthreads();
#pragma unroll
    for (int it = 0; it < LI; ++it) {
      const int row = ld_row + it * (kThreads / BK);
      as[row * LD + ld_k] = a_r[it];
      bs[row * LD + ld_k] = b_r[it];
    }
    __syncthreads();
    if (k0 + BK < N) fetch(k0 + BK);
#pragma unroll
    for (int j = 0; j < BK / 8; ++j) {
      float4 av[2], bv[2];
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        av[u] = *reinterpret_cast<const float4*>(as + (wi + 32 * u + l32) * LD + 8 * j + 4 * lh);
        bv[u] = *reinterpret_cast<const float4*>(bs + (wj + 32 * u + l32) * LD + 8 * j + 4 * lh);
      }
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int v = 0; v < 2; ++v) {
          acc[u][v] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[u].x, bv[v].x, acc[u][v], 0, 0, 0);
          acc[u][v] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[u].y, bv[v].y, acc[u][v], 0, 0, 0);
          acc[u][v] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[u].z, bv[v].z, acc[u][v], 0, 0, 0);
          acc[u][v] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[u].w, bv[v].w, acc[u][v], 0, 0, 0);
        }
    }
  }
#pragma unroll
  for (int u = 0; u < 2; ++u)
#pragma unroll
    for (int v = 0; v < 2; ++v) {
      const int j = j0 + wj + 32 * v + l32;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int i = i0 + wi + 32 * u + acc_row(r, lh);
        if (i < N && j < N) x[plane + (size_t)i * N + j] = acc[u][v][r];
      }
    }
}

__global__ __launch_bounds__(kThreads) void trimul_out_f32(TrimulF32 p, int groups) {
  __shared__ float zn[kP][kMaxC];
  __shared__ float xs[kP][kMaxC];
  __shared__ float xo[kP][kMaxC];
  const int N = p.N, C = p.C, CH = p.CH;
  const int g = blockIdx.x % groups, i = (blockIdx.x / groups) % N, b = blockIdx.x / (groups * N);
  const int j0 = g * kP;
  auto zrow = [&](int pos) -> const float* {
    const int j = j0 + pos;
    return j < N ? p.z + b * p.zc.stride_b + i * p.zc.stride_r + j * p.zc.stride_k : nullptr;
  };
  layer_norm_rows(zrow, p.ln_in_w, p.ln_in_b, C, zn);
  for (int idx = threadIdx.x; idx < kP * CH; idx += kThreads) {
    const int pos = idx % kP, c = idx / kP, j = j0 + pos;
    xs[pos][c] = j < N ? p.x[(((size_t)b * CH + c) * N + i) * N + j] : 0.f;
  }
  __syncthreads();
  layer_norm_rows([&](int pos) -> const float* { return j0 + pos < N ? xs[pos] : nullptr; }, p.ln_out_w, p.ln_out_b,
                  CH, xo);
  __syncthreads();
  for (int idx = threadIdx.x; idx < kP * C; idx += kThreads) {
    const int pos = idx / C, co = idx % C, j = j0 + pos;
    if (j >= N) continue;
    float res = dot_row(xo[pos], p.w_z + co * CH, CH) * sigmoid_f32(dot_row(zn[pos], p.w_g + co * C, C));
    const size_t o = b * p.zc.stride_b + i * p.zc.stride_r + j * p.zc.stride_k + co;
    if (p.add_residual) res = p.z[o] + res;
    p.out[o] = res;
  }
}


// the two position-wise passes of the triangle multiplication on the matrix pipe: 32 positions of
// one row per work-group
__global__ __launch_bounds__(kThreads) void trimul_proj_mm_f32(TrimulF32 p, int groups) {
  extern __shared__ float smem[];
  const int N = p.N, C = p.C, CH = p.CH, ldx = C + 4;
  float* xn = smem;              // [kTP][ldx]
  float* msk = smem + kTP * ldx; // [kTP]
  const int g = blockIdx.x % groups, r = (blockIdx.x / groups) % N, b = blockIdx.x / (groups * N);
  const int k0 = g * kTP;
  layer_norm_tile(
      [&](int pos) -> const float* {
        const int k = k0 + pos;
        return k < N ? p.z + b * p.zv.stride_b + r * p.zv.stride_r + k * p.zv.stride_k : nullptr;
      },
      p.ln_in_w, p.ln_in_b, C, xn, ldx);
  if (threadIdx.x < kTP) {
    const int k = k0 + threadIdx.x;
    msk[threadIdx.x] = (k < N && p.mask) ? p.mask[b * p.mv.stride_b + r * p.mv.stride_r + k * p.mv.stride_k] : 1.f;
  }
  __syncthreads();
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, l32 = lane & 31, lh = lane >> 5;
  const int n_ot = (CH + 31) / 32;
  const int k = k0 + l32;  // lanes = positions: a and b are written k-contiguous
  const float m = msk[l32];
  for (int t = wave; t < 2 * n_ot; t += kThreads / 64) {
    const int pair = t / n_ot, o0 = 32 * (t - pair * n_ot);
    const float* const W[2] = {pair ? p.w_bg : p.w_ag, pair ? p.w_bp : p.w_ap};
    f32x16_t acc[2];
    linear_tiles<2, true>(xn, ldx, W, o0, CH, C, acc);
    float* dst = pair ? p.b : p.a;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int c = o0 + acc_row(v, lh);
      // mask * sigmoid(gate) * projection, in the reference's order of multiplication
      if (c < CH && k < N) dst[(((size_t)b * CH + c) * N + r) * N + k] = m * sigmoid_hw_f32(acc[0][v]) * acc[1][v];
    }
  }
}

__global__ __launch_bounds__(kThreads) void trimul_out_mm_f32(TrimulF32 p, int groups) {
  extern __shared__ float smem[];
  const int N = p.N, C = p.C, CH = p.CH, ldc = C + 4, ldh = CH + 4;
  float* zn = smem;             // [kTP][ldc]  LayerNorm(z)
  float* xs = zn + kTP * ldc;   // [kTP][ldh]  x gathered from the channel-major planes
  float* xo = xs + kTP * ldh;   // [kTP][ldh]  LayerNorm(x)
  const int g = blockIdx.x % groups, i = (blockIdx.x / groups) % N, b = blockIdx.x / (groups * N);
  const int j0 = g * kTP;
  layer_norm_tile(
      [&](int pos) -> const float* {
        const int j = j0 + pos;
        return j < N ? p.z + b * p.zc.stride_b + i * p.zc.stride_r + j * p.zc.stride_k : nullptr;
      },
      p.ln_in_w, p.ln_in_b, C, zn, ldc);
  for (int idx = threadIdx.x; idx < kTP * CH; idx += kThreads) {
    const int pos = idx % kTP, c = idx / kTP, j = j0 + pos;
    xs[pos * ldh + c] = j < N ? p.x[(((size_t)b * CH + c) * N + i) * N + j] : 0.f;
  }
  __syncthreads();
  layer_norm_tile([&](int pos) -> const float* { return j0 + pos < N ? xs + pos * ldh : nullptr; }, p.ln_out_w,
                  p.ln_out_b, CH, xo, ldh);
  __syncthreads();
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, l32 = lane & 31, lh = lane >> 5;
  const int n_ot = (C + 31) / 32;
  for (int t = wave; t < n_ot; t += kThreads / 64) {
    const int o0 = 32 * t, co = o0 + l32;  // lanes = output channels: rows of out are written contiguously
    const float* const Wz[1] = {p.w_z};
    const float* const Wg[1] = {p.w_g};
    f32x16_t lin[1], gate[1];
    linear_tiles<1, false>(xo, ldh, Wz, o0, C, CH, lin);
    linear_tiles<1, false>(zn, ldc, Wg, o0, C, C, gate);
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int j = j0 + acc_row(v, lh);
      if (co < C && j < N) {
        float res = lin[0][v] * sigmoid_hw_f32(gate[0][v]);
        const size_t o = b * p.zc.stride_b + i * p.zc.stride_r + j * p.zc.stride_k + co;
        if (p.add_residual) res = p.z[o] + res;
        p.out[o] = res;
      }
    }
  }
}

// The same two passes on split operands (channel counts that are multiples of 16), 32 * XT positions
// per work-group.  WIDE: more than 128 channels on either side (two output tiles per wave).  FAST:
// channel counts in multiples of 64 and 8-byte aligned rows; a work-group whose positions all lie
// below N then stores without lane conditions, from one address per lane plus wave-uniform offsets.
// SPLIT: a and b leave as bf16 terms in the k-panel layout of the split-operand contraction.
template <int XT, int PT, bool FAST, bool SPLIT>
__global__ __launch_bounds__(kThreads * PT) void trimul_proj_x3_f32(TrimulF32 p, int groups) {
  extern __shared__ float smem[];
  constexpr int TPX = 32 * XT * PT, NT = kThreads * PT;
  const int N = p.N, C = p.C, CH = p.CH;
  const TileX3 xn = make_tile_x3(smem, C, TPX);
  float* msk = reinterpret_cast<float*>(reinterpret_cast<char*>(smem) + tile_bytes_x3(C, TPX));  // [TPX]
  // the PT groups of four waves take PT consecutive rows r of the same 32 XT columns k: in the
  // k-panel layout of a and b these are contiguous, PT x 64 bytes per channel and term
  constexpr int KT = 32 * XT;
  const int row_groups = (N + PT - 1) / PT;
  const int g = blockIdx.x % groups, r0 = ((blockIdx.x / groups) % row_groups) * PT, b = blockIdx.x / (groups * row_groups);
  const int k0 = g * KT;
  layer_norm_tile_x3<XT * PT, FAST, NT>(
      [&](int pos, bool& valid) -> const float* {
        const int r = r0 + pos / KT, k = k0 + pos % KT;
        valid = r < N && k < N;
        return p.z + b * p.zv.stride_b + (r < N ? r : N - 1) * p.zv.stride_r + (k < N ? k : N - 1) * p.zv.stride_k;
      },
      p.ln_in_w, p.ln_in_b, C, xn, NoExtra{});
  if (threadIdx.x < TPX) {
    const int r = r0 + threadIdx.x / KT, k = k0 + threadIdx.x % KT;
    msk[threadIdx.x] =
        (r < N && k < N && p.mask) ? p.mask[b * p.mv.stride_b + r * p.mv.stride_r + k * p.mv.stride_k] : 1.f;
  }
  __syncthreads();
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63, l32 = lane & 31,
            lh = lane >> 5;
  const int jw = wave & 3, pb = KT * (wave >> 2);  // this wave's share of the output tiles and its positions
  const int r = r0 + (wave >> 2);                  // (its row)
  if (r >= N) return;                              // no barrier follows
  const bool whole = k0 + KT <= N;
  const int n_ot = (CH + 31) / 32;
  const size_t NN = (size_t)N * N;
  for (int t = jw; t < 2 * n_ot; t += 4) {
    const int pair = t / n_ot, o0 = 32 * (t - pair * n_ot);
    const WeightX3 W[2] = {pair ? p.s_bg : p.s_ag, pair ? p.s_bp : p.s_ap};
    f32x16_t acc[2][XT];
    if (SPLIT) {
      // Channels in the lanes, positions in the registers: registers 8 t .. 8 t + 7 of a lane are the k
      // 16 t + 8 (e >> 2) + 4 lh + (e & 3) of its channel, stored as the 8 consecutive columns
      // 16 t + 8 lh .. + 7 of the panel row (16 bytes per term).  a and b use the same order inside
      // every 16 columns, which is all a sum over k needs.  Positions past N were normalised to zero
      // rows: they store zeros, the k padding of the panel.
      linear_tiles_x3<2, XT, false>(xn.at(pb), W, o0, C, acc);
      const int c = o0 + l32;
      const size_t chan = (size_t)p.Np * p.Np;  // elements per channel
#pragma unroll
      for (int xt = 0; xt < XT; ++xt) {
        if (k0 + 32 * xt >= p.Np || !(FAST || c < CH)) continue;
        bf16_t* lp = (pair ? p.bs : p.as) + ((size_t)b * CH + c) * chan +
                     ((size_t)((k0 + 32 * xt) >> 5) * p.Np + r) * 32 + 8 * lh;
#pragma unroll
        for (int st = 0; st < 2; ++st) {
          float x[8];
#pragma unroll
          for (int a = 0; a < 2; ++a) {
            const float4 m4 = *reinterpret_cast<const float4*>(msk + pb + 32 * xt + 16 * st + 8 * a + 4 * lh);
            const float m[4] = {m4.x, m4.y, m4.z, m4.w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const int v = 8 * st + 4 * a + e;
              x[4 * a + e] = m[e] * sigmoid_hw_f32(acc[0][xt][v]) * acc[1][xt][v];
            }
          }
          u32x4_t h, mid, lo;
          split8(x, h, mid, lo);
          *reinterpret_cast<u32x4_t*>(lp + 16 * st) = h;
          *reinterpret_cast<u32x4_t*>(lp + p.ab_plane + 16 * st) = mid;
          *reinterpret_cast<u32x4_t*>(lp + 2 * p.ab_plane + 16 * st) = lo;
        }
      }
      continue;
    }
    linear_tiles_x3<2, XT, true>(xn.at(pb), W, o0, C, acc);
    float* dst = pair ? p.b : p.a;
#pragma unroll
    for (int xt = 0; xt < XT; ++xt) {
      const int k = k0 + 32 * xt + l32;
      const float m = msk[pb + 32 * xt + l32];
      if (FAST && whole) {
        float* lp = dst + (((size_t)b * CH + o0) * N + r) * N + (size_t)(4 * lh) * NN + k;
#pragma unroll
        for (int v = 0; v < 16; ++v)
          lp[(size_t)(8 * (v >> 2) + (v & 3)) * NN] = m * sigmoid_hw_f32(acc[0][xt][v]) * acc[1][xt][v];
      } else {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int c = o0 + acc_row(v, lh);
          if (c < CH && k < N)
            dst[(((size_t)b * CH + c) * N + r) * N + k] = m * sigmoid_hw_f32(acc[0][xt][v]) * acc[1][xt][v];
        }
      }
    }
  }
}

// Contraction on split operands: x[b][c][i][j] = sum_k a[b][c][i][k] b[b][c][j][k] in fp32, six bf16
// products per k-step.  Work-group = 8 waves (4 x 2) = a 256 x 128 tile of one channel, a wave owns
// 64 x 64 (2 x 2 MFMA tiles).  Per 32-wide k-panel the three terms of the tile's a rows and b rows
// travel global -> LDS with direct-to-LDS buffer loads, one panel ahead, into double buffers; one
// vmcnt(0) + barrier per panel.  A row of a panel is 64 bytes = 4 chunks of 16 bytes; chunk c of row
// r is stored at position c ^ ((r >> 2) & 3), so that the 8 lanes of an operand read (8 rows, same
// chunk) fall into different banks; the swizzle is applied on the global side.
constexpr int kCtM = 256, kCtN = 128;
constexpr int kCtASlots = kCtM * 4, kCtBSlots = kCtN * 4;      // per term and stage, in 16-byte slots
constexpr int kCtStage = 3 * (kCtASlots + kCtBSlots);
constexpr size_t kContractX3Lds = (size_t)2 * kCtStage * 16;

__global__ __launch_bounds__(512) void trimul_contract_x3_f32(TrimulF32 p, int tiles_m, int tiles_n, int total,
                                                               int per_xcd) {
  extern __shared__ u32x4_t lds4[];
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int lane = tid & 63, l32 = lane & 31, lh = lane >> 5;
  const int N = p.N, Np = p.Np, panels = Np / 32;
  const int logical = xcd_logical_block(blockIdx.x, per_xcd);
  if (logical >= total) return;  // the whole work-group leaves together
  const int tn = logical % tiles_n, tm = (logical / tiles_n) % tiles_m, bc = logical / (tiles_n * tiles_m);
  const int i0 = tm * kCtM, j0 = tn * kCtN;
  const size_t chan = (size_t)Np * Np;
  // one descriptor per term and side over the channel's plane
  __amdgpu_buffer_rsrc_t a_rsrc[3], b_rsrc[3];
#pragma unroll
  for (int pl = 0; pl < 3; ++pl) {
    a_rsrc[pl] = buffer_rsrc(p.as + pl * p.ab_plane + bc * chan, chan * sizeof(bf16_t));
    b_rsrc[pl] = buffer_rsrc(p.bs + pl * p.ab_plane + bc * chan, chan * sizeof(bf16_t));
  }
  // slot t of a stage's a (b) part holds chunk (t & 3) ^ ((row >> 2) & 3) of tile row t >> 2; wave w
  // fills a slots 128 w .. + 127 (two instructions) and b slots 64 w .. + 63 of each term
  uint32_t a_off[2], b_off;
#pragma unroll
  for (int n = 0; n < 2; ++n) {
    const int t = 128 * wave + 64 * n + lane, row = t >> 2, c = (t & 3) ^ ((row >> 2) & 3);
    a_off[n] = (uint32_t)(((i0 + row) * 32 + 8 * c) * sizeof(bf16_t));
  }
  {
    const int t = 64 * wave + lane, row = t >> 2, c = (t & 3) ^ ((row >> 2) & 3);
    b_off = (uint32_t)(((j0 + row) * 32 + 8 * c) * sizeof(bf16_t));
  }
  auto issue_loads = [&](int panel, int buf) {  // buf is a constant at every call site
    u32x4_t* st = lds4 + buf * kCtStage;
    const int soff = panel * Np * 32 * (int)sizeof(bf16_t);
#pragma unroll
    for (int pl = 0; pl < 3; ++pl) {
#pragma unroll
      for (int n = 0; n < 2; ++n)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(a_rsrc[pl], (void OF3_LDS_AS*)(st + pl * kCtASlots + 128 * wave + 64 * n), 16,
                                                 a_off[n], soff, 0, 0);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(b_rsrc[pl], (void OF3_LDS_AS*)(st + 3 * kCtASlots + pl * kCtBSlots + 64 * wave),
                                               16, b_off, soff, 0, 0);
    }
  };
  f32x16_t acc[2][2];
#pragma unroll
  for (int mi = 0; mi < 2; ++mi)
#pragma unroll
    for (int ni = 0; ni < 2; ++ni) acc[mi][ni] = zero16();
  const int key = (l32 >> 2) & 3;
  auto panel_products = [&](int buf) {
    const u32x4_t* sa = lds4 + buf * kCtStage + (64 * wm + l32) * 4;
    const u32x4_t* sb = lds4 + buf * kCtStage + 3 * kCtASlots + (64 * wn + l32) * 4;
#pragma unroll
    for (int st = 0; st < 2; ++st) {
      const int c = (2 * st + lh) ^ key;
      u32x4_t ao[2][3], bo[2][3];
#pragma unroll
      for (int pl = 0; pl < 3; ++pl) {
#pragma unroll
        for (int mi = 0; mi < 2; ++mi) ao[mi][pl] = sa[pl * kCtASlots + mi * 128 + c];
#pragma unroll
        for (int ni = 0; ni < 2; ++ni) bo[ni][pl] = sb[pl * kCtBSlots + ni * 128 + c];
      }
#pragma unroll
      for (int mi = 0; mi < 2; ++mi)
#pragma unroll
        for (int ni = 0; ni < 2; ++ni) {  // smallest terms first
          acc[mi][ni] = mfma_32x32x16(ao[mi][2], bo[ni][0], acc[mi][ni]);
          acc[mi][ni] = mfma_32x32x16(ao[mi][0], bo[ni][2], acc[mi][ni]);
          acc[mi][ni] = mfma_32x32x16(ao[mi][1], bo[ni][1], acc[mi][ni]);
          acc[mi][ni] = mfma_32x32x16(ao[mi][1], bo[ni][0], acc[mi][ni]);
          acc[mi][ni] = mfma_32x32x16(ao[mi][0], bo[ni][1], acc[mi][ni]);
          acc[mi][ni] = mfma_32x32x16(ao[mi][0], bo[ni][0], acc[mi][ni]);
        }
    }
  };
  issue_loads(0, 0);
  auto step = [&](int panel, int buf) {
    wait_vmcnt<0>();               // this wave's loads of the panel have landed ...
    __builtin_amdgcn_s_barrier();  // ... and everybody's; nobody reads the previous panel's buffers any more
    compiler_fence();
    issue_loads(panel + 1 < panels ? panel + 1 : panels - 1, buf ^ 1);
    panel_products(buf);
    compiler_fence();
  };
  for (int panel = 0; panel < panels; panel += 2) {
    step(panel, 0);
    if (panel + 1 < panels) step(panel + 1, 1);
  }
  wait_vmcnt<0>();  // the loads issued past the end must not outlive the work-group's LDS

  float* xc = p.x + (size_t)bc * N * N;
#pragma unroll
  for (int mi = 0; mi < 2; ++mi)
#pragma unroll
    for (int ni = 0; ni < 2; ++ni) {
      const int ib = i0 + 64 * wm + 32 * mi, j = j0 + 64 * wn + 32 * ni + l32;
      if (ib + 32 <= N && j0 + 64 * wn + 32 * ni + 32 <= N) {
        float* lp = xc + (size_t)(ib + 4 * lh) * N + j;
#pragma unroll
        for (int v = 0; v < 16; ++v) lp[(size_t)(8 * (v >> 2) + (v & 3)) * N] = acc[mi][ni][v];
      } else {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int i = ib + acc_row(v, lh);
          if (i < N && j < N) xc[(size_t)i * N + j] = acc[mi][ni][v];
        }
      }
    }
}

// Output pass.  The gate is computed first and kept in registers, so that LayerNorm(x) can take the
// place of LayerNorm(z) in LDS.  x is read channel-major straight into registers: thread (position
// pos = tid % TPX, channel group cg = tid / TPX) holds the channel pairs 2 cg + 2 CG e, + 1; the
// statistics of a position are summed over the channel groups through LDS.
template <int XT, int PT, bool WIDE, bool FAST>
__global__ __launch_bounds__(kThreads * PT) void trimul_out_x3_f32(TrimulF32 p, int groups) {
  extern __shared__ float smem[];
  constexpr int TPX = 32 * XT * PT, NT = kThreads * PT, CG = NT / TPX, XP = (WIDE ? 128 : 64) / CG, MAXT = WIDE ? 2 : 1;
  const int N = p.N, C = p.C, CH = p.CH;
  char* base = reinterpret_cast<char*>(smem);
  const TileX3 zn = make_tile_x3(base, C, TPX);   // LayerNorm(z), then
  const TileX3 xo = make_tile_x3(base, CH, TPX);  // LayerNorm(x) in the same memory
  const size_t tile_max = tile_bytes_x3(C > CH ? C : CH, TPX);
  float* red_s = reinterpret_cast<float*>(base + tile_max);  // [CG][TPX]
  float* red_q = red_s + NT;                                 // [CG][TPX]
  const int g = blockIdx.x % groups, i = (blockIdx.x / groups) % N, b = blockIdx.x / (groups * N);
  const int j0 = g * TPX;
  const bool whole = j0 + TPX <= N;
  const int xpos = threadIdx.x % TPX, cg = threadIdx.x / TPX;
  const bool xin = j0 + xpos < N;
  const size_t NN = (size_t)N * N;
  float xv[2 * XP];
  {
    const float* xp = p.x + (((size_t)b * CH + 2 * cg) * N + i) * N + j0 + xpos;
#pragma unroll
    for (int e = 0; e < XP; ++e) {
      const bool in = xin && 2 * cg + 2 * CG * e < CH;
      xv[2 * e] = in ? xp[(size_t)(2 * CG * e) * NN] : 0.f;
      xv[2 * e + 1] = in ? xp[(size_t)(2 * CG * e + 1) * NN] : 0.f;
    }
  }
  layer_norm_tile_x3<XT * PT, FAST, NT>(
      [&](int pos, bool& valid) -> const float* {
        const int j = j0 + pos;
        valid = j < N;
        return p.z + b * p.zc.stride_b + i * p.zc.stride_r + (j < N ? j : N - 1) * p.zc.stride_k;
      },
      p.ln_in_w, p.ln_in_b, C, zn, NoExtra{});
  __syncthreads();
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63, l32 = lane & 31,
            lh = lane >> 5;
  const int jw = wave & 3, pb = 32 * XT * (wave >> 2);  // this wave's share of the output tiles and its positions
  const int n_ot = (C + 31) / 32;
  f32x16_t gate[MAXT][1][XT];
#pragma unroll
  for (int u = 0; u < MAXT; ++u) {
    const int t = jw + 4 * u;
    if (t < n_ot) {
      const WeightX3 Wg[1] = {p.s_g};
      linear_tiles_x3<1, XT, false>(zn.at(pb), Wg, 32 * t, C, gate[u]);
    }
  }
  // LayerNorm over the channels of x
  {
    float s = 0.f;
#pragma unroll
    for (int e = 0; e < 2 * XP; ++e) s += xv[e];
    red_s[threadIdx.x] = s;
  }
  __syncthreads();  // also: every wave has finished reading zn
  float mean = 0.f;
#pragma unroll
  for (int c = 0; c < CG; ++c) mean += red_s[c * TPX + xpos];
  mean /= (float)CH;
  {
    float q = 0.f;
#pragma unroll
    for (int e = 0; e < XP; ++e)
      if (2 * cg + 2 * CG * e < CH) {
        const float d0 = xv[2 * e] - mean, d1 = xv[2 * e + 1] - mean;
        q += d0 * d0;
        q += d1 * d1;
      }
    red_q[threadIdx.x] = q;
  }
  __syncthreads();
  float var = 0.f;
#pragma unroll
  for (int c = 0; c < CG; ++c) var += red_q[c * TPX + xpos];
  const float rstd = 1.0f / sqrtf(var / (float)CH + kEps);
#pragma unroll
  for (int e = 0; e < XP; ++e) {
    const int c = 2 * cg + 2 * CG * e;
    if (c < CH)
      xo.store2(xpos, c, xin ? (xv[2 * e] - mean) * rstd * p.ln_out_w[c] + p.ln_out_b[c] : 0.f,
                xin ? (xv[2 * e + 1] - mean) * rstd * p.ln_out_w[c + 1] + p.ln_out_b[c + 1] : 0.f);
  }
  __syncthreads();
#pragma unroll
  for (int u = 0; u < MAXT; ++u) {
    const int t = jw + 4 * u;
    if (t < n_ot) {
      const int o0 = 32 * t, co = o0 + l32;
      const WeightX3 Wz[1] = {p.s_z};
      f32x16_t lin[1][XT];
      linear_tiles_x3<1, XT, false>(xo.at(pb), Wz, o0, CH, lin);
#pragma unroll
      for (int xt = 0; xt < XT; ++xt) {
        if (FAST && whole) {
          const size_t lo = b * p.zc.stride_b + i * p.zc.stride_r + (size_t)(j0 + pb + 32 * xt + 4 * lh) * p.zc.stride_k + co;
          const float* zp = p.z + lo;
          float* op = p.out + lo;
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            const size_t vo = (size_t)(8 * (v >> 2) + (v & 3)) * p.zc.stride_k;
            float res = lin[0][xt][v] * sigmoid_hw_f32(gate[u][0][xt][v]);
            if (p.add_residual) res = zp[vo] + res;
            op[vo] = res;
          }
        } else {
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            const int j = j0 + pb + 32 * xt + acc_row(v, lh);
            if (co < C && j < N) {
              float res = lin[0][xt][v] * sigmoid_hw_f32(gate[u][0][xt][v]);
              const size_t o = b * p.zc.stride_b + i * p.zc.stride_r + j * p.zc.stride_k + co;
              if (p.add_residual) res = p.z[o] + res;
              p.out[o] = res;
            }
          }
        }
      }
    }
  }
}

// ---- triangle attention ----------------------------------------------------------------------
struct TriattnF32 {
  const float *x, *mask;
  PairView xv, mv;
  const float *ln_w, *ln_b, *w_q, *w_k, *w_v, *w_b, *w_g, *w_o;
  WeightX3 s_q, s_k, s_v, s_g, s_o;  // split copies (the *_x3 kernels only)
  float *q, *k, *v, *tb, *o, *out;
  // q, k and v^T split into three bf16 terms and stored as MFMA operands (the split-operand core only):
  // the 16 bytes of lane l for step s of 32-position tile t of (b, i, h) are slot
  // (((b N + i) H + h) * Jp / 32 + t) * steps + s) * 64 + l of a plane.  q and k have D / 16 steps (16
  // head channels each) and planes of qk_plane elements; v^T always has two steps (16 keys each) of 32
  // rows, the rows from D on being zero, and planes of v_plane elements
  bf16_t *qs, *ks, *vs;
  long qk_plane, v_plane;
  int Jp;  // N rounded up to whole 32-position tiles
  int B, N, C, H, D, add_residual;
  float inf;
};

__global__ __launch_bounds__(kThreads) void triattn_proj_f32(TriattnF32 p, int groups) {
  __shared__ float xn[kP][kMaxC];
  const int N = p.N, C = p.C, H = p.H, D = p.D, HD = H * D;
  const int g = blockIdx.x % groups, i = (blockIdx.x / groups) % N, b = blockIdx.x / (groups * N);
  const int j0 = g * kP;
  layer_norm_rows(
      [&](int pos) -> const float* {
        const int j = j0 + pos;
        return j < N ? p.x + b * p.xv.stride_b + i * p.xv.stride_r + j * p.xv.stride_k : nullptr;
      },
      p.ln_w, p.ln_b, C, xn);
  __syncthreads();
  const float scale = 1.0f / sqrtf((float)D);
  for (int idx = threadIdx.x; idx < kP * (3 * HD + H); idx += kThreads) {
    const int pos = idx % kP, ch = idx / kP, j = j0 + pos;
    if (j >= N) continue;
    if (ch < 3 * HD) {
      const int which = ch / HD, hd = ch % HD, h = hd / D, d = hd % D;
      const float* w = (which == 0 ? p.w_q : which == 1 ? p.w_k : p.w_v) + hd * C;
      float val = dot_row(xn[pos], w, C);
      if (which == 0) val = val * scale;  // q / sqrt(c) after the projection (attention.py:283-284)
      float* dst = which == 0 ? p.q : which == 1 ? p.k : p.v;
      dst[((((size_t)b * N + i) * H + h) * N + j) * D + d] = val;
    } else {
      const int h = ch - 3 * HD;
      p.tb[(((size_t)b * H + h) * N + i) * N + j] = dot_row(xn[pos], p.w_b + h * C, C);
    }
  }
}

__global__ __launch_bounds__(kThreads) void triattn_proj_mm_f32(TriattnF32 p, int groups) {
  extern __shared__ float smem[];
  const int N = p.N, C = p.C, H = p.H, D = p.D, HD = H * D, ldx = C + 4;
  float* xn = smem;  // [kTP][ldx]
  const int g = blockIdx.x % groups, i = (blockIdx.x / groups) % N, b = blockIdx.x / (groups * N);
  const int j0 = g * kTP;
  layer_norm_tile(
      [&](int pos) -> const float* {
        const int j = j0 + pos;
        return j < N ? p.x + b * p.xv.stride_b + i * p.xv.stride_r + j * p.xv.stride_k : nullptr;
      },
      p.ln_w, p.ln_b, C, xn, ldx);
  __syncthreads();
  const float scale = 1.0f / sqrtf((float)D);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, l32 = lane & 31, lh = lane >> 5;
  const int n_ot = (HD + 31) / 32, n_bt = (H + 31) / 32;
  for (int t = wave; t < n_ot + n_bt; t += kThreads / 64) {
    if (t < n_ot) {
      // q, k, v: lanes = head channels (d-contiguous stores)
      const int o0 = 32 * t, hd = o0 + l32, h = hd / D, d = hd - h * D;
      const float* const W[3] = {p.w_q, p.w_k, p.w_v};
      f32x16_t acc[3];
      linear_tiles<3, false>(xn, ldx, W, o0, HD, C, acc);
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int j = j0 + acc_row(v, lh);
        if (hd < HD && j < N) {
          const size_t o = ((((size_t)b * N + i) * H + h) * N + j) * D + d;
          p.q[o] = acc[0][v] * scale;  // q / sqrt(c) after the projection (attention.py:283-284)
          p.k[o] = acc[1][v];
          p.v[o] = acc[2][v];
        }
      }
    } else {
      // triangle bias: lanes = positions (j-contiguous stores)
      const int o0 = 32 * (t - n_ot), j = j0 + l32;
      const float* const W[1] = {p.w_b};
      f32x16_t acc[1];
      linear_tiles<1, true>(xn, ldx, W, o0, H, C, acc);
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int h = o0 + acc_row(v, lh);
        if (h < H && j < N) p.tb[(((size_t)b * H + h) * N + i) * N + j] = acc[0][v];
      }
    }
  }
}

__global__ __launch_bounds__(kThreads) void triattn_out_mm_f32(TriattnF32 p, int groups) {
  extern __shared__ float smem[];
  const int N = p.N, C = p.C, HD = p.H * p.D, ldx = C + 4, ldh = HD + 4;
  float* xn = smem;             // [kTP][ldx]
  float* og = xn + kTP * ldx;   // [kTP][ldh]  gated attention output
  const int g = blockIdx.x % groups, i = (blockIdx.x / groups) % N, b = blockIdx.x / (groups * N);
  const int j0 = g * kTP;
  layer_norm_tile(
      [&](int pos) -> const float* {
        const int j = j0 + pos;
        return j < N ? p.x + b * p.xv.stride_b + i * p.xv.stride_r + j * p.xv.stride_k : nullptr;
      },
      p.ln_w, p.ln_b, C, xn, ldx);
  __syncthreads();
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, l32 = lane & 31, lh = lane >> 5;
  for (int t = wave; t < (HD + 31) / 32; t += kThreads / 64) {
    const int o0 = 32 * t, hd = o0 + l32;
    const float* const W[1] = {p.w_g};
    f32x16_t gate[1];
    linear_tiles<1, false>(xn, ldx, W, o0, HD, C, gate);
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int pos = acc_row(v, lh), j = j0 + pos;
      if (hd < HD)
        og[pos * ldh + hd] = j < N ? p.o[(((size_t)b * N + i) * N + j) * HD + hd] * sigmoid_hw_f32(gate[0][v]) : 0.f;
    }
  }
  __syncthreads();
  for (int t = wave; t < (C + 31) / 32; t += kThreads / 64) {
    const int o0 = 32 * t, co = o0 + l32;
    const float* const W[1] = {p.w_o};
    f32x16_t acc[1];
    linear_tiles<1, false>(og, ldh, W, o0, C, HD, acc);
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int j = j0 + acc_row(v, lh);
      if (co < C && j < N) {
        float res = acc[0][v];
        const size_t o = b * p.xv.stride_b + i * p.xv.stride_r + j * p.xv.stride_k + co;
        if (p.add_residual) res = p.x[o] + res;
        p.out[o] = res;
      }
    }
  }
}

// The two position-wise passes of the attention on split operands (channel counts that are multiples
// of 16), 32 * XT positions per work-group.  The H rows of the triangle bias are too few for a matrix
// tile: they are fp32 dot products taken on the normalised row while it is in registers.
// SPLIT (head width 32 or 16): q, k and v leave as operands of the split-operand core instead of fp32 arrays.
// A 32-column tile of the projections is one head, or two of width 16.  q and k are computed with the head channels in
// the accumulator rows and the positions in the lanes, v the other way round: in both cases registers
// 8 s .. 8 s + 7 of a lane are its operand for step s (q, k: head channels 16 s + 4 lh + r and
// 16 s + 8 + 4 lh + r, the same for both, so the order inside the dot product does not matter;
// v: the keys the core's S^T accumulator holds in the same registers).
template <int XT, int PT, bool SPLIT, bool FAST>
__global__ __launch_bounds__(kThreads * PT) void triattn_proj_x3_f32(TriattnF32 p, int groups) {
  extern __shared__ float smem[];
  constexpr int TPX = 32 * XT * PT, NT = kThreads * PT;
  const int N = p.N, C = p.C, H = p.H, D = p.D, HD = H * D;
  const TileX3 xn = make_tile_x3(smem, C, TPX);
  float* tbs = reinterpret_cast<float*>(reinterpret_cast<char*>(smem) + tile_bytes_x3(C, TPX));  // [H][TPX]
  const int g = blockIdx.x % groups, i = (blockIdx.x / groups) % N, b = blockIdx.x / (groups * N);
  const int j0 = g * TPX;
  const int l = threadIdx.x & 31;
  layer_norm_tile_x3<XT * PT, FAST, NT>(
      [&](int pos, bool& valid) -> const float* {
        const int j = j0 + pos;
        valid = j < N;
        return p.x + b * p.xv.stride_b + i * p.xv.stride_r + (j < N ? j : N - 1) * p.xv.stride_k;
      },
      p.ln_w, p.ln_b, C, xn, [&](int pos, const float(&y)[8]) {
        for (int h = 0; h < H; ++h) {
          const float* wb = p.w_b + h * C + 2 * l;
          float d = 0.f;
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (FAST ? 64 * e < C : 2 * l + 64 * e < C) {
              d += y[2 * e] * wb[64 * e];
              d += y[2 * e + 1] * wb[64 * e + 1];
            }
#pragma unroll
          for (int o = 16; o > 0; o >>= 1) d += __shfl_xor(d, o, 32);
          if (l == 0) tbs[h * TPX + pos] = d;
        }
      });
  __syncthreads();
  for (int idx = threadIdx.x; idx < H * TPX; idx += NT) {
    const int h = idx / TPX, j = j0 + idx % TPX;
    if (SPLIT) {
      // rows padded to whole 32-position tiles; positions past N were normalised to zero rows and store 0
      if (j < p.Jp) p.tb[(((size_t)b * H + h) * N + i) * p.Jp + j] = tbs[idx];
    } else if (j < N) {
      p.tb[(((size_t)b * H + h) * N + i) * N + j] = tbs[idx];
    }
  }
  const float scale = 1.0f / sqrtf((float)D);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63, l32 = lane & 31,
            lh = lane >> 5;
  const int jw = wave & 3, pb = 32 * XT * (wave >> 2);  // this wave's share of the output tiles and its positions
  for (int t = jw; t < (HD + 31) / 32; t += 4) {
    const int o0 = 32 * t;
    if (SPLIT) {
      // positions past N were normalised to zero rows: their q, k and v are zeros, and are stored.
      // Head width 32: tile t is head t.  Head width 16: tile t is heads 2 t and 2 t + 1; step st of the
      // q / k tile is the one step of head 2 t + st, and lane l32 of the v tile is row l32 % 16 of head
      // 2 t + l32 / 16, whose rows 16 .. 31 are written as zeros.
      const bool narrow = D == 16;
      const int nt = p.Jp / 32, jt0 = (j0 + pb) / 32;
      const size_t bi = (size_t)b * N + i;
      auto split_regs = [&](const f32x16_t& acc, int st, float mul, u32x4_t& h, u32x4_t& m, u32x4_t& lo) {
        float x[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) x[e] = acc[8 * st + e] * mul;
        split8(x, h, m, lo);
      };
      auto store_qk = [&](bf16_t* dst, const f32x16_t& acc, int xt, float mul) {
        if (j0 + pb + 32 * xt >= p.Jp) return;  // a tile past the padded row (XT > 1 only)
        const long plane = p.qk_plane / 8;
#pragma unroll
        for (int st = 0; st < 2; ++st) {
          const size_t slot = narrow ? ((bi * H + 2 * t + st) * nt + jt0 + xt) * 64 + lane
                                     : (((bi * H + t) * nt + jt0 + xt) * 2 + st) * 64 + lane;
          u32x4_t* d4 = reinterpret_cast<u32x4_t*>(dst) + slot;
          u32x4_t h, m, lo;
          split_regs(acc, st, mul, h, m, lo);
          d4[0] = h;
          d4[plane] = m;
          d4[2 * plane] = lo;
        }
      };
      auto store_v = [&](const f32x16_t& acc, int xt) {
        if (j0 + pb + 32 * xt >= p.Jp) return;
        const long plane = p.v_plane / 8;
        const int head = narrow ? 2 * t + (l32 >> 4) : t, vrow = narrow ? (l32 & 15) : l32;
#pragma unroll
        for (int st = 0; st < 2; ++st) {
          u32x4_t* d4 = reinterpret_cast<u32x4_t*>(p.vs) + (((bi * H + head) * nt + jt0 + xt) * 2 + st) * 64 + vrow + 32 * lh;
          u32x4_t h, m, lo;
          split_regs(acc, st, 1.f, h, m, lo);
          d4[0] = h;
          d4[plane] = m;
          d4[2 * plane] = lo;
          if (narrow) {
            const u32x4_t zero = {0u, 0u, 0u, 0u};
            d4[16] = zero;
            d4[plane + 16] = zero;
            d4[2 * plane + 16] = zero;
          }
        }
      };
      {
        const WeightX3 W[2] = {p.s_q, p.s_k};
        f32x16_t acc[2][XT];
        linear_tiles_x3<2, XT, true>(xn.at(pb), W, o0, C, acc);
#pragma unroll
        for (int xt = 0; xt < XT; ++xt) {
          store_qk(p.qs, acc[0][xt], xt, scale);  // q / sqrt(c) after the projection (attention.py:283-284)
          store_qk(p.ks, acc[1][xt], xt, 1.f);
        }
      }
      {
        const WeightX3 W[1] = {p.s_v};
        f32x16_t acc[1][XT];
        linear_tiles_x3<1, XT, false>(xn.at(pb), W, o0, C, acc);
#pragma unroll
        for (int xt = 0; xt < XT; ++xt) store_v(acc[0][xt], xt);
      }
    } else {
      const int hd = o0 + l32, h = hd / D, d = hd - h * D;
      const WeightX3 W[3] = {p.s_q, p.s_k, p.s_v};
      f32x16_t acc[3][XT];
      linear_tiles_x3<3, XT, false>(xn.at(pb), W, o0, C, acc);
#pragma unroll
      for (int xt = 0; xt < XT; ++xt)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int j = j0 + pb + 32 * xt + acc_row(v, lh);
          if (hd < HD && j < N) {
            const size_t o = ((((size_t)b * N + i) * H + h) * N + j) * D + d;
            p.q[o] = acc[0][xt][v] * scale;  // q / sqrt(c) after the projection (attention.py:283-284)
            p.k[o] = acc[1][xt][v];
            p.v[o] = acc[2][xt][v];
          }
        }
    }
  }
}

// Output pass: the gate stays in registers until every wave has finished with LayerNorm(x), then the
// gated attention output takes its place in LDS.
template <int XT, int PT, bool WIDE, bool FAST>
__global__ __launch_bounds__(kThreads * PT) void triattn_out_x3_f32(TriattnF32 p, int groups) {
  extern __shared__ float smem[];
  constexpr int TPX = 32 * XT * PT, NT = kThreads * PT, MAXT = WIDE ? 2 : 1;
  const int N = p.N, C = p.C, HD = p.H * p.D;
  const TileX3 xn = make_tile_x3(smem, C, TPX);
  const TileX3 og = make_tile_x3(smem, HD, TPX);  // gated attention output, in the same memory
  const int g = blockIdx.x % groups, i = (blockIdx.x / groups) % N, b = blockIdx.x / (groups * N);
  const int j0 = g * TPX;
  layer_norm_tile_x3<XT * PT, FAST, NT>(
      [&](int pos, bool& valid) -> const float* {
        const int j = j0 + pos;
        valid = j < N;
        return p.x + b * p.xv.stride_b + i * p.xv.stride_r + (j < N ? j : N - 1) * p.xv.stride_k;
      },
      p.ln_w, p.ln_b, C, xn, NoExtra{});
  __syncthreads();
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63, l32 = lane & 31,
            lh = lane >> 5;
  const int jw = wave & 3, pb = 32 * XT * (wave >> 2);  // this wave's share of the output tiles and its positions
  const bool whole = j0 + TPX <= N;
  const int n_gt = (HD + 31) / 32;
  f32x16_t gate[MAXT][1][XT];
#pragma unroll
  for (int u = 0; u < MAXT; ++u) {
    const int t = jw + 4 * u;
    if (t < n_gt) {
      const WeightX3 W[1] = {p.s_g};
      linear_tiles_x3<1, XT, false>(xn.at(pb), W, 32 * t, C, gate[u]);
    }
  }
  __syncthreads();
#pragma unroll
  for (int u = 0; u < MAXT; ++u) {
    const int t = jw + 4 * u, hd = 32 * t + l32;
    if (t < n_gt && hd < HD) {
#pragma unroll
      for (int xt = 0; xt < XT; ++xt) {
        if (whole) {
          const float* op = p.o + (((size_t)b * N + i) * N + j0 + pb + 32 * xt + 4 * lh) * HD + hd;
#pragma unroll
          for (int v = 0; v < 16; ++v)
            og.store(pb + 32 * xt + acc_row(v, lh), hd, op[(8 * (v >> 2) + (v & 3)) * HD] * sigmoid_hw_f32(gate[u][0][xt][v]));
        } else {
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            const int pos = pb + 32 * xt + acc_row(v, lh), j = j0 + pos;
            og.store(pos, hd,
                     j < N ? p.o[(((size_t)b * N + i) * N + j) * HD + hd] * sigmoid_hw_f32(gate[u][0][xt][v]) : 0.f);
          }
        }
      }
    }
  }
  __syncthreads();
  for (int t = jw; t < (C + 31) / 32; t += 4) {
    const int o0 = 32 * t, co = o0 + l32;
    const WeightX3 W[1] = {p.s_o};
    f32x16_t acc[1][XT];
    linear_tiles_x3<1, XT, false>(og.at(pb), W, o0, HD, acc);
#pragma unroll
    for (int xt = 0; xt < XT; ++xt) {
      if (FAST && whole) {
        const size_t lo = b * p.xv.stride_b + i * p.xv.stride_r + (size_t)(j0 + pb + 32 * xt + 4 * lh) * p.xv.stride_k + co;
        const float* xp = p.x + lo;
        float* op = p.out + lo;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const size_t vo = (size_t)(8 * (v >> 2) + (v & 3)) * p.xv.stride_k;
          float res = acc[0][xt][v];
          if (p.add_residual) res = xp[vo] + res;
          op[vo] = res;
        }
      } else {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int j = j0 + pb + 32 * xt + acc_row(v, lh);
          if (co < C && j < N) {
            float res = acc[0][xt][v];
            const size_t o = b * p.xv.stride_b + i * p.xv.stride_r + j * p.xv.stride_k + co;
            if (p.add_residual) res = p.x[o] + res;
            p.out[o] = res;
          }
        }
      }
    }
  }
}

// Attention core on split operands, head width 16 * STEPS (32 or 16; the narrow head leaves half of the
// O^T tile's rows unused).  Work-group = 8 waves = 4 consecutive rows i x 2
// halves of one (head, 128-query range); a wave owns 64 queries (two 32-query tiles) of one row.
//   S^T = K Q^T  (rows = keys, columns = queries), six bf16 products per k-step, started from the
//                triangle bias (the accumulator is loaded with it; logits stay in natural units, not
//                pre-multiplied by log2(e): a row of masked keys has to lose its logits against -1e9 at
//                the reference's granularity, or it averages other keys than the reference does); the mask bias of a key tile rides
//                on one more k-step, A = [hi, mid, lo, 0 ...] of the key's bias split exactly into
//                three bf16 terms, B = [1, 1, 1, 0 ...], taken only by tiles with a masked or padded key
//   O^T = V^T P^T, the weights split in registers straight from the S^T accumulator into B operands
// Per 32-key tile the work-group brings in the bias slice of its query range (it does not depend on
// i: shared by the four rows) and each row's K and V^T operands (shared by the row's two waves) with
// direct-to-LDS buffer loads, one tile ahead, into double buffers: no registers are held for data in
// flight, and the only wait is one vmcnt(0) + barrier per key tile, a whole tile of arithmetic after
// the loads were issued.  The bias slice is XOR-swizzled on the global side (a lane picks which
// 16-byte chunk it fetches for its fixed LDS slot).  Softmax as in the bf16 core: a first pass with
// the offset 0 for every query that leaves out key tiles whose keys are all masked or padded, and a
// second pass with running maxima for the work-groups whose row sums say the first was not exact;
// keys past N carry a mask bias of -inf.
constexpr int kXRows = 4;
constexpr int kXTbSlots = 128 * 8;                     // bias slice [128 queries][32 keys] fp32 in 16-byte slots
constexpr int kXKvSlots = 12 * 64;                     // K step 0, 1 (h m l each), then V^T step 0, 1
constexpr size_t kCoreX3Lds = (size_t)(2 * kXTbSlots + 2 * kXRows * kXKvSlots) * 16;

template <int STEPS>
__global__ __launch_bounds__(512) void triattn_core_x3_f32(TriattnF32 p, int n_qc, int n_rg, int total, int per_xcd) {
  constexpr int QT = 2, D = 16 * STEPS;
  extern __shared__ u32x4_t lds4[];
  u32x4_t* tb_lds = lds4;                   // [2][kXTbSlots]
  u32x4_t* kv_lds = lds4 + 2 * kXTbSlots;   // [kXRows][2][kXKvSlots]
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int row = wave >> 1, qh = wave & 1;
  const int lane = tid & 63, l32 = lane & 31, lh = lane >> 5;
  const int N = p.N, H = p.H, Jp = p.Jp, nt = Jp / 32;
  const int logical = xcd_logical_block(blockIdx.x, per_xcd);
  if (logical >= total) return;  // the whole work-group leaves together
  const int qc = logical % n_qc, rg = (logical / n_qc) % n_rg, bh = logical / (n_qc * n_rg);
  const int i_raw = rg * kXRows + row;
  const bool row_valid = i_raw < N;  // wave-uniform; idle waves still take part in the loads and barriers
  const int i = row_valid ? i_raw : N - 1;
  const int b = bh / H, h = bh % H;
  const int q0 = qc * 128 + 64 * qh;
  const size_t bih = ((size_t)b * N + i) * H + h;
  const long plane = p.qk_plane / 8;  // in 16-byte slots
  const u32x4_t* Q = reinterpret_cast<const u32x4_t*>(p.qs) + bih * nt * (64 * STEPS) + lane;
  const float* tbp = p.tb + ((size_t)b * H + h) * N * Jp;  // rows padded to Jp, zeros past N
  const int nkt = nt;

  u32x4_t qop[QT][STEPS][3];
#pragma unroll
  for (int qt = 0; qt < QT; ++qt) {
    const int jt = q0 / 32 + qt < nt ? q0 / 32 + qt : nt - 1;  // tiles past the end: computed, not stored
#pragma unroll
    for (int st = 0; st < STEPS; ++st)
#pragma unroll
      for (int pl = 0; pl < 3; ++pl) qop[qt][st][pl] = Q[pl * plane + (jt * STEPS + st) * 64];
  }

  // bias slice: instruction n of wave w fills slots 64 (2 w + n) .. + 63; slot t holds chunk
  // (t & 7) ^ ((q >> 1) & 7) of query q = t >> 3 of the work-group's range
  uint32_t tb_off[2];
#pragma unroll
  for (int n = 0; n < 2; ++n) {
    const int t = 64 * (2 * wave + n) + lane;
    const int qloc = t >> 3, chunk = (t & 7) ^ ((qloc >> 1) & 7);
    int qrow = qc * 128 + qloc;
    qrow = qrow < N ? qrow : N - 1;
    tb_off[n] = (uint32_t)(((size_t)qrow * Jp + 4 * chunk) * sizeof(float));
  }
  // this wave's share of its row's tile: the K operands (first wave of the row) or the V^T operands,
  // one descriptor per term (a plane can be larger than a descriptor's range)
  const int kv_steps = qh ? 2 : STEPS;  // 1-KB operands per key tile and term
  const long kv_plane = qh ? p.v_plane : p.qk_plane;
  const bf16_t* kvp = (qh ? p.vs : p.ks) + bih * Jp * (16 * kv_steps);
  const size_t kv_bytes = (size_t)Jp * (32 * kv_steps);
  const __amdgpu_buffer_rsrc_t kv_rsrc[3] = {buffer_rsrc(kvp, kv_bytes), buffer_rsrc(kvp + kv_plane, kv_bytes),
                                             buffer_rsrc(kvp + 2 * kv_plane, kv_bytes)};
  const __amdgpu_buffer_rsrc_t tb_rsrc = buffer_rsrc(tbp, (size_t)N * Jp * sizeof(float));
  const uint32_t lane_off = lane * 16;
  u32x4_t* kv_row = kv_lds + row * (2 * kXKvSlots);
  auto issue_loads = [&](int kt, int buf) {  // buf is a constant at every call site
    u32x4_t* tdst = tb_lds + buf * kXTbSlots + 128 * wave;
    u32x4_t* kdst = kv_row + buf * kXKvSlots + 6 * 64 * qh;
#pragma unroll
    for (int n = 0; n < 2; ++n)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(tb_rsrc, (void OF3_LDS_AS*)(tdst + 64 * n), 16, tb_off[n],
                                               kt * (32 * (int)sizeof(float)), 0, 0);
#pragma unroll
    for (int st = 0; st < 2; ++st)
      if (st < kv_steps) {  // wave-uniform
#pragma unroll
        for (int pl = 0; pl < 3; ++pl)
          __builtin_amdgcn_raw_ptr_buffer_load_lds(kv_rsrc[pl], (void OF3_LDS_AS*)(kdst + (st * 3 + pl) * 64), 16, lane_off,
                                                   (kt * kv_steps + st) * 1024, 0, 0);
      }
  };
  // mask value of key 32 kt + l32 (clamped to a real key; some bias value when there is no mask: not used)
  const float* mrow = p.mask ? p.mask + b * p.mv.stride_b + i * p.mv.stride_r : tbp;
  const long mstep = p.mask ? p.mv.stride_k : 1;
  auto load_mask = [&](int kt) {
    const int k = kt * 32 + l32 < N ? kt * 32 + l32 : N - 1;
    return mrow[k * mstep];
  };
  auto mask_bias = [&](int kt, float mv) {
    return kt * 32 + l32 < N ? (p.mask ? p.inf * (mv - 1.f) : 0.f) : -__builtin_inff();
  };
  // the mask-bias k-step on the 8-deep MFMA (two registers per operand): lanes 0..31 hold k = 0..3
  auto mask_step = [&](float mb, f32x16_t acc) {
    const bool lo = lh == 0;
    const uint32_t hi_bits = __float_as_uint(mb) & 0xffff0000u;
    const float r1 = __builtin_isinf(mb) ? 0.f : mb - __uint_as_float(hi_bits);  // exact
    const uint32_t mid_bits = __float_as_uint(r1) & 0xffff0000u;
    const float r2 = r1 - __uint_as_float(mid_bits);  // exact, at most 8 significant bits
    const u32x2_t a_op = {lo ? ((hi_bits >> 16) | mid_bits) : 0u, lo ? (__float_as_uint(r2) >> 16) : 0u};
    const u32x2_t b_op = {lo ? 0x3F803F80u : 0u, lo ? 0x3F80u : 0u};
    return mfma_32x32x8(a_op, b_op, acc);
  };

  f32x16_t oacc[QT];
  float m_run[QT], l_run[QT], l_tot[QT];
  const int tb_key = (l32 >> 1) & 7;

  // a wave of a row past the end, or whose queries all lie past the end, still takes part in the loads and
  // barriers of its work-group but leaves the arithmetic out; so does a 32-query tile past the end
  const bool wave_has_work = row_valid && q0 < N;
  // track = false: the first pass, offset 0 for every query (no maximum, no rescaling); track = true: running maxima
  auto tile = [&](auto track, int buf, float mb) {
    constexpr bool kTrack = decltype(track)::value;
    if (!wave_has_work) return;
    // first pass: a tile whose keys are all masked or padded adds exp(-1e9 + logit) = 0 exactly to every sum
    if (!kTrack && __builtin_amdgcn_ballot_w64(mb > -1e8f) == 0) return;
    const bool has_mb = __builtin_amdgcn_ballot_w64(mb != 0.f) != 0;
    const u32x4_t* kvb = kv_row + buf * kXKvSlots + lane;
    const u32x4_t* tbuf = tb_lds + buf * kXTbSlots + (64 * qh + l32) * 8;
    u32x4_t kop[STEPS][3];
#pragma unroll
    for (int st = 0; st < STEPS; ++st)
#pragma unroll
      for (int pl = 0; pl < 3; ++pl) kop[st][pl] = kvb[(st * 3 + pl) * 64];
#pragma unroll
    for (int qt = 0; qt < QT; ++qt) {
      if (qt > 0 && q0 + 32 * qt >= N) continue;
      f32x16_t s;
#pragma unroll
      for (int a = 0; a < 4; ++a) {  // registers 4 a .. 4 a + 3: keys 8 a + 4 lh .. + 3 = chunk 2 a + lh
        const u32x4_t t = tbuf[qt * 256 + ((2 * a + lh) ^ tb_key)];
#pragma unroll
        for (int e = 0; e < 4; ++e) s[4 * a + e] = __uint_as_float(t[e]);
      }
      if (has_mb) s = mask_step(mb, s);
#pragma unroll
      for (int st = 0; st < STEPS; ++st) {  // smallest terms first
        s = mfma_32x32x16(kop[st][2], qop[qt][st][0], s);
        s = mfma_32x32x16(kop[st][0], qop[qt][st][2], s);
        s = mfma_32x32x16(kop[st][1], qop[qt][st][1], s);
        s = mfma_32x32x16(kop[st][1], qop[qt][st][0], s);
        s = mfma_32x32x16(kop[st][0], qop[qt][st][1], s);
        s = mfma_32x32x16(kop[st][0], qop[qt][st][0], s);
      }
      float lsum = 0.f;
      if constexpr (kTrack) {
        float cmax = s[0];
#pragma unroll
        for (int v = 1; v < 16; ++v) cmax = fmaxf(cmax, s[v]);
        cmax = fmaxf(cmax, __shfl_xor(cmax, 32, 64));  // the other half of the query's keys
        const float m_new = fmaxf(m_run[qt], cmax);    // finite: every tile holds a key below N
        const float alpha = __builtin_amdgcn_exp2f((m_run[qt] - m_new) * kLog2eF32);
        m_run[qt] = m_new;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          s[v] = __builtin_amdgcn_exp2f((s[v] - m_new) * kLog2eF32);
          lsum += s[v];
        }
        l_run[qt] = l_run[qt] * alpha + lsum;
#pragma unroll
        for (int v = 0; v < 16; ++v) oacc[qt][v] *= alpha;
      } else {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          s[v] = __builtin_amdgcn_exp2f(s[v] * kLog2eF32);
          lsum += s[v];
        }
        l_run[qt] += lsum;
      }
#pragma unroll
      for (int st = 0; st < 2; ++st) {
        float x[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) x[e] = s[8 * st + e];
        u32x4_t ph, pm, pl;
        split8(x, ph, pm, pl);
        const u32x4_t vh = kvb[(6 + st * 3) * 64], vm = kvb[(7 + st * 3) * 64], vl = kvb[(8 + st * 3) * 64];
        oacc[qt] = mfma_32x32x16(vl, ph, oacc[qt]);
        oacc[qt] = mfma_32x32x16(vh, pl, oacc[qt]);
        oacc[qt] = mfma_32x32x16(vm, pm, oacc[qt]);
        oacc[qt] = mfma_32x32x16(vm, ph, oacc[qt]);
        oacc[qt] = mfma_32x32x16(vh, pm, oacc[qt]);
        oacc[qt] = mfma_32x32x16(vh, ph, oacc[qt]);
      }
    }
  };

  auto pass = [&](auto track) {
#pragma unroll
    for (int qt = 0; qt < QT; ++qt) {
      oacc[qt] = zero16();
      m_run[qt] = -__builtin_inff();
      l_run[qt] = 0.f;
    }
    float mv_next = load_mask(0);
    issue_loads(0, 0);
    auto step = [&](int kt, int buf) {  // buf is a constant at both call sites: LDS addresses are immediates
      wait_vmcnt<0>();               // this wave's loads of tile kt (and its mask values) have landed ...
      __builtin_amdgcn_s_barrier();  // ... and everybody's; nobody reads tile kt - 1's buffers any more
      compiler_fence();
      const float mb = mask_bias(kt, mv_next);
      const int ktn = kt + 1 < nkt ? kt + 1 : nkt - 1;
      mv_next = load_mask(ktn);
      issue_loads(ktn, buf ^ 1);
      tile(track, buf, mb);
      compiler_fence();
    };
    for (int kt = 0; kt < nkt; kt += 2) {
      step(kt, 0);
      if (kt + 1 < nkt) step(kt + 1, 1);
    }
    wait_vmcnt<0>();  // the loads issued past the end must not outlive the pass (or the work-group's LDS)
#pragma unroll
    for (int qt = 0; qt < QT; ++qt) l_tot[qt] = l_run[qt] + __shfl_xor(l_run[qt], 32, 64);
  };

  // First pass: offset 0 for every query (any common offset gives the same softmax): a logit costs one
  // multiplication, one exp2 and one addition, no maximum and no rescaling of the accumulator.  It is exact
  // whenever the exponentials neither overflowed nor lost the row's largest terms, which the row sum tells:
  // 2^-60 <= sum <= 2^60 (an overflow leaves +inf, a row of masked keys leaves 0).  A work-group with a query
  // outside that range (its loads and barriers are collective) runs the pass again with running maxima.
  pass(std::false_type{});
  {
    bool bad = false;
#pragma unroll
    for (int qt = 0; qt < QT; ++qt) {
      const bool in_range = l_tot[qt] >= 0x1p-60f && l_tot[qt] <= 0x1p60f;  // false for NaN too
      bad |= row_valid && (q0 + 32 * qt + l32 < N) && !in_range;
    }
    if (__syncthreads_or(bad)) pass(std::true_type{});
  }

  if (row_valid) {
#pragma unroll
    for (int qt = 0; qt < QT; ++qt) {
      const int q = q0 + 32 * qt + l32;
      if (q >= N) continue;
      const float inv = 1.0f / l_tot[qt];
      float* dst = p.o + ((((size_t)b * N + i) * N + q) * H + h) * D + 4 * lh;
#pragma unroll
      for (int a = 0; a < D / 8; ++a)  // registers 4 a .. 4 a + 3 are head channels 8 a + 4 lh .. + 3
        *reinterpret_cast<float4*>(dst + 8 * a) = make_float4(oacc[qt][4 * a] * inv, oacc[qt][4 * a + 1] * inv,
                                                              oacc[qt][4 * a + 2] * inv, oacc[qt][4 * a + 3] * inv);
    }
  }
}

// Attention core on the fp32 matrix pipe.  Work-group = 4 waves = 128 queries of one (b, i, h), a
// wave owns 32 of them; keys in chunks of 32 through LDS, and with them the [128 queries x 32 keys]
// slice of the triangle bias (loaded row-wise, 128 contiguous bytes per query); online softmax.
//   S^T = K Q^T   rows = keys, columns = queries: a lane ends with 16 logits of one query
//   O^T = V^T P^T rows = head channels; the weights go from the S^T accumulator registers straight
//                 into the B operand: MFMA step v pairs the keys acc_row(v, 0) and acc_row(v, 1)
// Logits in the reference's order: q.k, then the mask bias, then the triangle bias.
template <int DP>
__global__ __launch_bounds__(kThreads, 2) void triattn_core_f32(TriattnF32 p, int qgroups) {
  static_assert(DP % 8 == 0 && DP <= 64, "head widths up to 64, rounded up to a multiple of 8");
  constexpr int KC = 32, LD = DP + 4;  // padded rows: the 16 lanes of a float4 read phase cover all banks
  constexpr int OB = (DP + 31) / 32;   // 32-channel blocks of the output
  const int D = p.D;                   // the head width itself: channels D .. DP - 1 are zeros in LDS
  static_assert(kThreads == 256, "four waves of 32 queries");
  __shared__ __align__(16) float ks[KC * LD];
  __shared__ float vs[KC * LD], mbs[KC];
  __shared__ float tbs[128][KC + 1];
  const int N = p.N, H = p.H;
  const int qg = blockIdx.x % qgroups, h = (blockIdx.x / qgroups) % H, i = (blockIdx.x / (qgroups * H)) % N,
            b = blockIdx.x / (qgroups * H * N);
  const int lane = threadIdx.x & 63, l32 = lane & 31, lh = lane >> 5;
  const int qloc = 32 * (threadIdx.x >> 6) + l32;  // this lane's query among the work-group's 128
  const int qi = qg * 128 + qloc;
  const bool active = qi < N;
  const size_t bih = (((size_t)b * N + i) * H + h) * N;
  // B operands of S^T: MFMA step 4j+e pairs d = 8j+e (lanes 0-31) with d = 8j+4+e (lanes 32-63)
  float qv[DP / 8][4];
#pragma unroll
  for (int j = 0; j < DP / 8; ++j)
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int d = 8 * j + 4 * lh + e;
      qv[j][e] = active && d < D ? p.q[(bih + qi) * D + d] : 0.f;
    }
  f32x16_t oacc[OB];
#pragma unroll
  for (int ob = 0; ob < OB; ++ob) oacc[ob] = zero16();
  const float* tbq = p.tb + (((size_t)b * H + h) * N + (size_t)qg * 128) * N;  // row of query qg*128
  float m = -__builtin_inff(), l = 0.f;
  // a chunk's K, V, bias slice and mask values travel global -> registers while the previous chunk
  // is being computed, and registers -> LDS between two barriers
  constexpr int KVI = KC * DP / kThreads, TBI = 128 * KC / kThreads;
  float k_r[KVI], v_r[KVI], tb_r[TBI], mb_r = 0.f;
  auto fetch = [&](int k0) {
#pragma unroll
    for (int it = 0; it < KVI; ++it) {
      const int e = threadIdx.x + it * kThreads, kk = e / DP, d = e % DP;
      const bool in = k0 + kk < N && d < D;
      k_r[it] = in ? p.k[(bih + k0 + kk) * D + d] : 0.f;
      v_r[it] = in ? p.v[(bih + k0 + kk) * D + d] : 0.f;
    }
#pragma unroll
    for (int it = 0; it < TBI; ++it) {
      const int e = threadIdx.x + it * kThreads, r = e / KC, c = e % KC;
      tb_r[it] = (qg * 128 + r < N && k0 + c < N) ? tbq[(size_t)r * N + k0 + c] : 0.f;
    }
    if (threadIdx.x < KC) {
      const int kx = k0 + threadIdx.x;
      float mv = 1.f;
      if (kx < N && p.mask) mv = p.mask[b * p.mv.stride_b + i * p.mv.stride_r + kx * p.mv.stride_k];
      mb_r = p.inf * (mv - 1.f);
    }
  };
  fetch(0);
  for (int k0 = 0; k0 < N; k0 += KC) {
    __syncthreads();
#pragma unroll
    for (int it = 0; it < KVI; ++it) {
      const int e = threadIdx.x + it * kThreads, kk = e / DP, d = e % DP;
      ks[kk * LD + d] = k_r[it];
      vs[kk * LD + d] = v_r[it];
    }
#pragma unroll
    for (int it = 0; it < TBI; ++it) {
      const int e = threadIdx.x + it * kThreads;
      tbs[e / KC][e % KC] = tb_r[it];
    }
    if (threadIdx.x < KC) mbs[threadIdx.x] = mb_r;
    __syncthreads();
    if (k0 + KC < N) fetch(k0 + KC);
    const int kn = N - k0 < KC ? N - k0 : KC;
    f32x16_t s = zero16();
#pragma unroll
    for (int j = 0; j < DP / 8; ++j) {
      const float4 kk = *reinterpret_cast<const float4*>(ks + l32 * LD + 8 * j + 4 * lh);
      s = __builtin_amdgcn_mfma_f32_32x32x2f32(kk.x, qv[j][0], s, 0, 0, 0);
      s = __builtin_amdgcn_mfma_f32_32x32x2f32(kk.y, qv[j][1], s, 0, 0, 0);
      s = __builtin_amdgcn_mfma_f32_32x32x2f32(kk.z, qv[j][2], s, 0, 0, 0);
      s = __builtin_amdgcn_mfma_f32_32x32x2f32(kk.w, qv[j][3], s, 0, 0, 0);
    }
    float cmax = -__builtin_inff();
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int kk = acc_row(v, lh);
      float a = s[v] + mbs[kk];
      a = a + tbs[qloc][kk];
      a = kk < kn ? a : -__builtin_inff();
      s[v] = a;
      cmax = fmaxf(cmax, a);
    }
    cmax = fmaxf(cmax, __shfl_xor(cmax, 32, 64));  // the other half of the query's keys
    const float m_new = fmaxf(m, cmax);
    // exp(x) as the hardware's exp2(x * log2(e)): about 2 ulp for the arguments of a softmax, far
    // inside the 1e-4 bound, and a sixth of expf's instructions
    const float alpha = __builtin_amdgcn_exp2f((m - m_new) * kLog2eF32);
    l *= alpha;
#pragma unroll
    for (int ob = 0; ob < OB; ++ob)
#pragma unroll
      for (int v = 0; v < 16; ++v) oacc[ob][v] *= alpha;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const float pw = __builtin_amdgcn_exp2f((s[v] - m_new) * kLog2eF32);
      l += pw;
      s[v] = pw;
    }
#pragma unroll
    for (int ob = 0; ob < OB; ++ob) {
      const int ch = 32 * ob + l32 < DP ? 32 * ob + l32 : DP - 1;  // rows past D are computed and dropped
#pragma unroll
      for (int v = 0; v < 16; ++v)
        oacc[ob] = __builtin_amdgcn_mfma_f32_32x32x2f32(vs[acc_row(v, lh) * LD + ch], s[v], oacc[ob], 0, 0, 0);
    }
    m = m_new;
  }
  l += __shfl_xor(l, 32, 64);
  if (active) {
    const float inv = 1.0f / l;
    float* dst = p.o + ((((size_t)b * N + i) * N + qi) * H + h) * D;
#pragma unroll
    for (int ob = 0; ob < OB; ++ob)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int ch = 32 * ob + acc_row(v, lh);
        if (ch < D) dst[ch] = oacc[ob][v] * inv;
      }
  }
}

__global__ __launch_bounds__(kThreads) void triattn_out_f32(TriattnF32 p, int groups) {
  __shared__ float xn[kP][kMaxC];
  __shared__ float og[kP][kMaxC];
  const int N = p.N, C = p.C, HD = p.H * p.D;
  const int g = blockIdx.x % groups, i = (blockIdx.x / groups) % N, b = blockIdx.x / (groups * N);
  const int j0 = g * kP;
  layer_norm_rows(
      [&](int pos) -> const float* {
        const int j = j0 + pos;
        return j < N ? p.x + b * p.xv.stride_b + i * p.xv.stride_r + j * p.xv.stride_k : nullptr;
      },
      p.ln_w, p.ln_b, C, xn);
  __syncthreads();
  for (int idx = threadIdx.x; idx < kP * HD; idx += kThreads) {
    const int pos = idx / HD, hd = idx % HD, j = j0 + pos;
    og[pos][hd] = j < N ? p.o[(((size_t)b * N + i) * N + j) * HD + hd] * sigmoid_f32(dot_row(xn[pos], p.w_g + hd * C, C))
                        : 0.f;
  }
  __syncthreads();
  for (int idx = threadIdx.x; idx < kP * C; idx += kThreads) {
    const int pos = idx / C, co = idx % C, j = j0 + pos;
    if (j >= N) continue;
    float res = dot_row(og[pos], p.w_o + co * HD, HD);
    const size_t o = b * p.xv.stride_b + i * p.xv.stride_r + j * p.xv.stride_k + co;
    if (p.add_residual) res = p.x[o] + res;
    p.out[o] = res;
  }
}

// ---- pair transition -------------------------------------------------------------------------
constexpr int kMaxHid = 1024;

struct TransitionF32 {
  const float *x, *mask;
  PairView xv, mv;
  const float *ln_w, *ln_b, *w_a, *w_b, *w_out;
  WeightX3 s_a, s_b, s_out;  // split copies (transition_x3_f32 only)
  float* out;
  int B, N, C, HID, add_residual;
};

// out = [x +] ((silu(xn Wa^T) * (xn Wb^T)) Wout^T) * mask for kP positions of one row
__global__ __launch_bounds__(kThreads) void transition_f32(TransitionF32 p, int groups) {
  __shared__ float xn[kP][kMaxC];
  __shared__ float hid[kP][kMaxHid];
  const int N = p.N, C = p.C, HID = p.HID;
  const int g = blockIdx.x % groups, i = (blockIdx.x / groups) % N, b = blockIdx.x / (groups * N);
  const int j0 = g * kP;
  layer_norm_rows(
      [&](int pos) -> const float* {
        const int j = j0 + pos;
        return j < N ? p.x + b * p.xv.stride_b + i * p.xv.stride_r + j * p.xv.stride_k : nullptr;
      },
      p.ln_w, p.ln_b, C, xn);
  __syncthreads();
  for (int idx = threadIdx.x; idx < kP * HID; idx += kThreads) {
    const int pos = idx / HID, hd = idx % HID;
    const float a = dot_row(xn[pos], p.w_a + (size_t)hd * C, C);
    const float bb = dot_row(xn[pos], p.w_b + (size_t)hd * C, C);
    hid[pos][hd] = (a * sigmoid_f32(a)) * bb;
  }
  __syncthreads();
  for (int idx = threadIdx.x; idx < kP * C; idx += kThreads) {
    const int pos = idx / C, co = idx % C, j = j0 + pos;
    if (j >= N) continue;
    float res = dot_row(hid[pos], p.w_out + (size_t)co * HID, HID);
    if (p.mask) res *= p.mask[b * p.mv.stride_b + i * p.mv.stride_r + j * p.mv.stride_k];
    const size_t o = b * p.xv.stride_b + i * p.xv.stride_r + j * p.xv.stride_k + co;
    if (p.add_residual) res = p.x[o] + res;
    p.out[o] = res;
  }
}

// the same on the matrix pipe, 32 positions per work-group.  The hidden dimension is walked in
// slices of `hchunk` (a multiple of 32): a slice of the hidden activations is computed into LDS and
// at once folded into the output accumulators, so that LDS holds one slice, not the whole hidden row
__global__ __launch_bounds__(kThreads) void transition_mm_f32(TransitionF32 p, int groups, int hchunk) {
  extern __shared__ float smem[];
  const int N = p.N, C = p.C, HID = p.HID, ldx = C + 4, ldh = hchunk + 4;
  float* xn = smem;             // [kTP][ldx]
  float* hid = xn + kTP * ldx;  // [kTP][ldh]
  const int g = blockIdx.x % groups, i = (blockIdx.x / groups) % N, b = blockIdx.x / (groups * N);
  const int j0 = g * kTP;
  layer_norm_tile(
      [&](int pos) -> const float* {
        const int j = j0 + pos;
        return j < N ? p.x + b * p.xv.stride_b + i * p.xv.stride_r + j * p.xv.stride_k : nullptr;
      },
      p.ln_w, p.ln_b, C, xn, ldx);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, l32 = lane & 31, lh = lane >> 5;
  // output tiles of this wave (C <= 256: at most two), accumulated over the hidden slices
  constexpr int kMaxOT = (kMaxC / 32 + kThreads / 64 - 1) / (kThreads / 64);
  f32x16_t out_acc[kMaxOT][1];
#pragma unroll
  for (int u = 0; u < kMaxOT; ++u) out_acc[u][0] = zero16();
  const int n_ot = (C + 31) / 32;
  for (int h0 = 0; h0 < HID; h0 += hchunk) {
    const int hn = HID - h0 < hchunk ? HID - h0 : hchunk;  // a multiple of 8
    __syncthreads();  // xn is complete (first slice); nobody reads the previous slice any more
    for (int t = wave; t < (hn + 31) / 32; t += kThreads / 64) {
      const int o0 = 32 * t, hd = o0 + l32;
      const float* const W[2] = {p.w_a + (size_t)h0 * C, p.w_b + (size_t)h0 * C};
      f32x16_t acc[2];
      linear_tiles<2, false>(xn, ldx, W, o0, hn, C, acc);
      if (hd < hn) {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const float a = acc[0][v];
          hid[acc_row(v, lh) * ldh + hd] = (a * sigmoid_hw_f32(a)) * acc[1][v];
        }
      }
    }
    __syncthreads();
#pragma unroll
    for (int u = 0; u < kMaxOT; ++u) {
      const int t = wave + u * (kThreads / 64);
      if (t < n_ot) {
        const float* const W[1] = {p.w_out + h0};
        linear_tiles<1, false, true>(hid, ldh, W, 32 * t, C, hn, out_acc[u], HID);
      }
    }
  }
#pragma unroll
  for (int u = 0; u < kMaxOT; ++u) {
    const int t = wave + u * (kThreads / 64), co = 32 * t + l32;
    if (t >= n_ot) continue;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int j = j0 + acc_row(v, lh);
      if (co < C && j < N) {
        float res = out_acc[u][0][v];
        if (p.mask) res *= p.mask[b * p.mv.stride_b + i * p.mv.stride_r + j * p.mv.stride_k];
        const size_t o = b * p.xv.stride_b + i * p.xv.stride_r + j * p.xv.stride_k + co;
        if (p.add_residual) res = p.x[o] + res;
        p.out[o] = res;
      }
    }
  }
}

// the same on split operands (C a multiple of 16, HID a multiple of 128), 32 positions per
// work-group, the hidden dimension in slices of 128: a wave computes one 32-column tile of the slice
// (both projections), writes silu(a) * b split into LDS, and adds the slice's share to its output tile
constexpr int kTrHC = 128;
template <bool WIDE, bool FAST>
__global__ __launch_bounds__(kThreads) void transition_x3_f32(TransitionF32 p, int groups) {
  extern __shared__ float smem[];
  constexpr int MAXT = WIDE ? 2 : 1;
  const int N = p.N, C = p.C, HID = p.HID;
  const TileX3 xn = make_tile_x3(smem, C, kTP);
  const TileX3 hid = make_tile_x3(reinterpret_cast<char*>(smem) + tile_bytes_x3(C, kTP), kTrHC, kTP);
  const int g = blockIdx.x % groups, i = (blockIdx.x / groups) % N, b = blockIdx.x / (groups * N);
  const int j0 = g * kTP;
  const bool whole = j0 + kTP <= N;
  layer_norm_tile_x3<1, FAST, kThreads>(
      [&](int pos, bool& valid) -> const float* {
        const int j = j0 + pos;
        valid = j < N;
        return p.x + b * p.xv.stride_b + i * p.xv.stride_r + (j < N ? j : N - 1) * p.xv.stride_k;
      },
      p.ln_w, p.ln_b, C, xn, NoExtra{});
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63, l32 = lane & 31,
            lh = lane >> 5;
  f32x16_t out_acc[MAXT][1][1];
#pragma unroll
  for (int u = 0; u < MAXT; ++u) out_acc[u][0][0] = zero16();
  const int n_ot = (C + 31) / 32;
  for (int h0 = 0; h0 < HID; h0 += kTrHC) {
    __syncthreads();  // xn is complete (first slice); nobody reads the previous slice any more
    {
      const WeightX3 W[2] = {p.s_a, p.s_b};
      f32x16_t acc[2][1];
      linear_tiles_x3<2, 1, false>(xn, W, h0 + 32 * wave, C, acc);
      const int hd = 32 * wave + l32;
#pragma unroll
      for (int v = 0; v < 16; v += 2) {  // positions acc_row(v) and acc_row(v) + 1 of this lane's hidden channel
        const float a0 = acc[0][0][v], a1 = acc[0][0][v + 1];
        hid.store(acc_row(v, lh), hd, (a0 * sigmoid_hw_f32(a0)) * acc[1][0][v]);
        hid.store(acc_row(v + 1, lh), hd, (a1 * sigmoid_hw_f32(a1)) * acc[1][0][v + 1]);
      }
    }
    __syncthreads();
#pragma unroll
    for (int u = 0; u < MAXT; ++u) {
      const int t = wave + 4 * u;
      if (t < n_ot) {
        const WeightX3 W[1] = {p.s_out};
        linear_tiles_x3<1, 1, false, true>(hid, W, 32 * t, kTrHC, out_acc[u], h0 / 16, HID / 16);
      }
    }
  }
#pragma unroll
  for (int u = 0; u < MAXT; ++u) {
    const int t = wave + 4 * u, co = 32 * t + l32;
    if (t >= n_ot) continue;
    if (FAST && whole) {
      const size_t lo = b * p.xv.stride_b + i * p.xv.stride_r + (size_t)(j0 + 4 * lh) * p.xv.stride_k + co;
      const float* mp = p.mask ? p.mask + b * p.mv.stride_b + i * p.mv.stride_r + (j0 + 4 * lh) * p.mv.stride_k : nullptr;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int dj = 8 * (v >> 2) + (v & 3);
        float res = out_acc[u][0][0][v];
        if (mp) res *= mp[dj * p.mv.stride_k];
        if (p.add_residual) res = p.x[lo + (size_t)dj * p.xv.stride_k] + res;
        p.out[lo + (size_t)dj * p.xv.stride_k] = res;
      }
    } else {
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int j = j0 + acc_row(v, lh);
        if (co < C && j < N) {
          float res = out_acc[u][0][0][v];
          if (p.mask) res *= p.mask[b * p.mv.stride_b + i * p.mv.stride_r + j * p.mv.stride_k];
          const size_t o = b * p.xv.stride_b + i * p.xv.stride_r + j * p.xv.stride_k + co;
          if (p.add_residual) res = p.x[o] + res;
          p.out[o] = res;
        }
      }
    }
  }
}

// ---- pair-bias projection ---------------------------------------------------------------------
struct PairBiasF32 {
  const float* z;
  PairView zv;
  const float *ln_w, *ln_b, *w;
  float* out;
  int B, N, C, H;
};

// out[b][h][i][j] = LN(z[b,i,j,:]) . w[h,:] for kP positions of one row
__global__ __launch_bounds__(kThreads) void pair_bias_f32(PairBiasF32 p, int groups) {
  __shared__ float xn[kP][kMaxC];
  __shared__ float zero_bias[kMaxC];
  const int N = p.N, C = p.C, H = p.H;
  const int g = blockIdx.x % groups, i = (blockIdx.x / groups) % N, b = blockIdx.x / (groups * N);
  const int j0 = g * kP;
  const float* lb = p.ln_b;
  if (!lb) {
    for (int c = threadIdx.x; c < C; c += kThreads) zero_bias[c] = 0.f;
    __syncthreads();
    lb = zero_bias;
  }
  layer_norm_rows(
      [&](int pos) -> const float* {
        const int j = j0 + pos;
        return j < N ? p.z + b * p.zv.stride_b + i * p.zv.stride_r + j * p.zv.stride_k : nullptr;
      },
      p.ln_w, lb, C, xn);
  __syncthreads();
  for (int idx = threadIdx.x; idx < kP * H; idx += kThreads) {
    const int pos = idx % kP, h = idx / kP, j = j0 + pos;
    if (j < N) p.out[(((size_t)b * H + h) * N + i) * N + j] = dot_row(xn[pos], p.w + (size_t)h * C, C);
  }
}

// the same on split operands (C a multiple of 16, H <= 32): one wave per 32 positions of a row and no
// other wave in the work-group, so that a CU holds as many independent tiles as its LDS has room for.
// The weights are few (H rows): a lane splits the eight values of its operand for a step on the way,
// the values of the next step being read while the current one is multiplied; head h is row h of
// the accumulator tile, the position its column: a head's 32 positions are one 128-byte store.
template <bool FAST>
__global__ __launch_bounds__(64) void pair_bias_x3_f32(PairBiasF32 p, int groups) {
  extern __shared__ float smem[];
  const int N = p.N, C = p.C, H = p.H;
  const TileX3 xn = make_tile_x3(smem, C, kTP);
  float* zero_bias = reinterpret_cast<float*>(reinterpret_cast<char*>(smem) + tile_bytes_x3(C, kTP));  // [C]
  const int g = blockIdx.x % groups, i = (blockIdx.x / groups) % N, b = blockIdx.x / (groups * N);
  const int j0 = g * kTP;
  const int lane = threadIdx.x, l32 = lane & 31, lh = lane >> 5;
  const float* lb = p.ln_b;
  if (!lb) {
    for (int c = lane; c < C; c += 64) zero_bias[c] = 0.f;
    __syncthreads();
    lb = zero_bias;
  }
  // this lane's weight operand: row min(l32, H - 1) (the rows from H on are dropped), k = 16 s + 8 lh ..
  const float* wrow = p.w + (size_t)(l32 < H ? l32 : H - 1) * C + 8 * lh;
  const bool wvec = (reinterpret_cast<uintptr_t>(p.w) & 15u) == 0;  // C % 16 == 0: every operand is then 16-byte aligned
  float wn[8];
  auto read_w = [&](int s) {
    if (wvec) {
      const float4 u = *reinterpret_cast<const float4*>(wrow + 16 * s), v = *reinterpret_cast<const float4*>(wrow + 16 * s + 4);
      wn[0] = u.x, wn[1] = u.y, wn[2] = u.z, wn[3] = u.w, wn[4] = v.x, wn[5] = v.y, wn[6] = v.z, wn[7] = v.w;
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) wn[e] = wrow[16 * s + e];
    }
  };
  read_w(0);
  layer_norm_tile_x3<1, FAST, 64>(
      [&](int pos, bool& valid) -> const float* {
        const int j = j0 + pos;
        valid = j < N;
        return p.z + b * p.zv.stride_b + i * p.zv.stride_r + (j < N ? j : N - 1) * p.zv.stride_k;
      },
      p.ln_w, lb, C, xn, NoExtra{});
  __syncthreads();
  const u32x4_t* xh = reinterpret_cast<const u32x4_t*>(xn.h + l32 * xn.ld + 8 * lh);
  const int xplane = xn.plane / 8;
  // the small terms and the large ones in accumulators of their own: two chains of dependent MFMAs
  // instead of one, and the small terms are summed among themselves before they meet the large ones
  f32x16_t acc = zero16(), acc_small = zero16();
  const int steps = C / 16;
  for (int s = 0; s < steps; ++s) {
    u32x4_t w_h, w_m, w_l;
    split8(wn, w_h, w_m, w_l);
    if (s + 1 < steps) read_w(s + 1);
    const u32x4_t x_h = xh[2 * s], x_m = xh[xplane + 2 * s], x_l = xh[2 * xplane + 2 * s];
    acc_small = mfma_32x32x16(w_l, x_h, acc_small);
    acc = mfma_32x32x16(w_m, x_h, acc);
    acc_small = mfma_32x32x16(w_h, x_l, acc_small);
    acc = mfma_32x32x16(w_h, x_m, acc);
    acc_small = mfma_32x32x16(w_m, x_m, acc_small);
    acc = mfma_32x32x16(w_h, x_h, acc);
  }
#pragma unroll
  for (int v = 0; v < 16; ++v) acc[v] += acc_small[v];
  const int j = j0 + l32;
  if (j < N) {
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int h = acc_row(v, lh);
      if (h < H) p.out[(((size_t)b * H + h) * N + i) * N + j] = acc[v];
    }
  }
}

// ---- template branch: closing LayerNorm of the stack and the mean / ReLU / linear_t tail -------
struct TemplateTailF32 {
  const float *t, *ln_w, *ln_b, *w;
  float* out;
  long P;
  int B, T, CT, CZ, apply_ln;
};

// kP positions per work-group: per template LayerNorm into xn, summed into acc (template order,
// like torch.sum), then / T, ReLU, and the C_z dot products
__global__ __launch_bounds__(kThreads) void template_tail_f32(TemplateTailF32 p, long groups) {
  __shared__ float xn[kP][kMaxC];
  __shared__ float acc[kP][kMaxC];
  const int CT = p.CT, CZ = p.CZ, T = p.T;
  const long g = blockIdx.x % groups;
  const int b = (int)(blockIdx.x / groups);
  const long p0 = g * kP;
  for (int idx = threadIdx.x; idx < kP * CT; idx += kThreads) acc[idx / CT][idx % CT] = 0.f;
  __syncthreads();
  for (int t = 0; t < T; ++t) {
    const float* plane = p.t + ((size_t)b * T + t) * p.P * CT;
    if (p.apply_ln) {
      layer_norm_rows([&](int pos) -> const float* { return p0 + pos < p.P ? plane + (p0 + pos) * CT : nullptr; },
                      p.ln_w, p.ln_b, CT, xn);
      __syncthreads();
      for (int idx = threadIdx.x; idx < kP * CT; idx += kThreads) acc[idx / CT][idx % CT] += xn[idx / CT][idx % CT];
    } else {
      for (int idx = threadIdx.x; idx < kP * CT; idx += kThreads) {
        const int pos = idx / CT, c = idx % CT;
        if (p0 + pos < p.P) acc[pos][c] += plane[(p0 + pos) * CT + c];
      }
    }
    __syncthreads();
  }
  for (int idx = threadIdx.x; idx < kP * CT; idx += kThreads) {
    const float m = acc[idx / CT][idx % CT] / (float)T;
    xn[idx / CT][idx % CT] = m > 0.f ? m : 0.f;
  }
  __syncthreads();
  for (int idx = threadIdx.x; idx < kP * CZ; idx += kThreads) {
    const int pos = idx / CZ, o = idx % CZ;
    if (p0 + pos < p.P) p.out[((size_t)b * p.P + p0 + pos) * CZ + o] = dot_row(xn[pos], p.w + (size_t)o * CT, CT);
  }
}

__global__ __launch_bounds__(kThreads) void layer_norm_f32(const float* __restrict__ x, const float* __restrict__ w,
                                                           const float* __restrict__ bsh, float* __restrict__ out,
                                                           long rows, int C) {
  __shared__ float xn[kP][kMaxC];
  const long r0 = (long)blockIdx.x * kP;
  layer_norm_rows([&](int pos) -> const float* { return r0 + pos < rows ? x + (r0 + pos) * C : nullptr; }, w, bsh, C, xn);
  __syncthreads();
  for (int idx = threadIdx.x; idx < kP * C; idx += kThreads) {
    const int pos = idx / C, c = idx % C;
    if (r0 + pos < rows) out[(r0 + pos) * C + c] = xn[pos][c];
  }
}


// ---- host side of the matrix-pipe kernels
size_t tile_bytes(int K) { return (size_t)kTP * (K + 4) * sizeof(float); }  // one LDS tile [kTP][K + 4]

bool aligned16(std::initializer_list<const void*> ptrs) {
  for (const void* q : ptrs)
    if (reinterpret_cast<uintptr_t>(q) % 16 != 0) return false;
  return true;
}

inline bool even_strides(const PairView& v) { return ((v.stride_b | v.stride_r | v.stride_k) & 1) == 0; }

// the largest tiles exceed the default dynamic LDS limit: raised to max_bytes once per device and
// kernel
constexpr size_t kLdsLimit = 160 * 1024;
#ifndef OF3_X3_XT
#define OF3_X3_XT 1
#endif
constexpr int kXT = OF3_X3_XT;  // 32-position tiles per wave of the split-operand passes
#ifndef OF3_X3_PT
#define OF3_X3_PT 2
#endif
constexpr int kPT = OF3_X3_PT;  // groups of four waves per work-group, each with its own positions: waves of different
                                // groups read the same weights at about the same time, once from L2
template <auto Kern>
hipError_t allow_lds(size_t max_bytes = 3 * (size_t)kTP * (kMaxC + 4) * sizeof(float)) {
  return allow_dynamic_lds<Kern>(max_bytes);
}

}  // namespace

hipError_t template_tail_fwd_f32(const TemplateTailF32Args& a, hipStream_t stream) {
  if (a.CT < 1 || a.CT > kMaxC || a.CZ < 1 || a.T < 1 || a.P < 1 || a.B < 1) return hipErrorInvalidValue;
  TemplateTailF32 p;
  p.t = a.t;
  p.ln_w = a.ln_w;
  p.ln_b = a.ln_b;
  p.w = a.w;
  p.out = a.out;
  p.P = a.P;
  p.B = a.B;
  p.T = a.T;
  p.CT = a.CT;
  p.CZ = a.CZ;
  p.apply_ln = a.apply_ln;
  const long groups = (a.P + kP - 1) / kP;
  const long blocks = groups * a.B;
  if (blocks > 0x7fffffffl) return hipErrorInvalidValue;
  hipLaunchKernelGGL(template_tail_f32, dim3((unsigned)blocks), dim3(kThreads), 0, stream, p, groups);
  return hipGetLastError();
}

hipError_t layer_norm_fwd_f32(const float* x, const float* w, const float* b, float* out, long rows, int C,
                              hipStream_t stream) {
  if (rows < 1 || C < 1 || C > kMaxC) return hipErrorInvalidValue;
  const long blocks = (rows + kP - 1) / kP;
  if (blocks > 0x7fffffffl) return hipErrorInvalidValue;
  hipLaunchKernelGGL(layer_norm_f32, dim3((unsigned)blocks), dim3(kThreads), 0, stream, x, w, b, out, rows, C);
  return hipGetLastError();
}

hipError_t trimul_fwd_f32(const TrimulF32Args& a, hipStream_t stream) {
  TrimulF32 p;
  p.z = a.z;
  p.mask = a.mask;
  p.zv = a.z_view;
  p.mv = a.mask_view;
  p.zc = a.z_canonical;
  p.ln_in_w = a.ln_in_w;
  p.ln_in_b = a.ln_in_b;
  p.ln_out_w = a.ln_out_w;
  p.ln_out_b = a.ln_out_b;
  p.w_ap = a.w_ap;
  p.w_ag = a.w_ag;
  p.w_bp = a.w_bp;
  p.w_bg = a.w_bg;
  p.w_g = a.w_g;
  p.w_z = a.w_z;
  p.a = a.a;
  p.b = a.b;
  p.x = a.x;
  p.out = a.out;
  p.B = a.B;
  p.N = a.N;
  p.C = a.C;
  p.CH = a.CH;
  p.add_residual = a.add_residual;
  const int groups = (a.N + kP - 1) / kP;
  const long blocks = (long)a.B * a.N * groups;
  if (a.C > kMaxC || a.CH > kMaxC || blocks > 0x7fffffffL) return hipErrorInvalidValue;
  const bool mm = a.C % 8 == 0 && a.CH % 8 == 0 &&
                  aligned16({a.w_ap, a.w_ag, a.w_bp, a.w_bg, a.w_g, a.w_z});
  const int mgroups = (a.N + kTP - 1) / kTP;
  const unsigned mblocks = (unsigned)((long)a.B * a.N * mgroups);
  // split-operand kernels for the position-wise passes: channel counts in multiples of 16 and room for
  // the split weights
  const bool x3 = a.C % 16 == 0 && a.CH % 16 == 0 && a.wsplit && aligned16({a.wsplit});
  // channel counts in multiples of 64 and rows of z on 8-byte boundaries in both frames
  const bool fast = a.C % 64 == 0 && a.CH % 64 == 0 && (reinterpret_cast<uintptr_t>(a.z) & 7u) == 0 &&
                    even_strides(a.z_view) && even_strides(a.z_canonical);
  // a and b as bf16 terms for the split-operand contraction (a channel's plane within 32-bit byte offsets)
  p.Np = (a.N + 31) / 32 * 32;
  p.ab_plane = (long)a.B * a.CH * p.Np * p.Np;
  p.as = static_cast<bf16_t*>(a.ab_split);
  p.bs = p.as + 3 * p.ab_plane;
  const bool split_ab = x3 && a.ab_split && aligned16({a.ab_split}) && (long)p.Np * p.Np * 2 <= 0x7fffffffL;
  const int xgroups = (a.N + 32 * kXT * kPT - 1) / (32 * kXT * kPT);
  const unsigned xblocks = (unsigned)((long)a.B * a.N * xgroups);
  if (x3) {
    WeightSplitter splitter(a.wsplit);
    splitter.add(a.w_ap, a.CH, a.C, p.s_ap);
    splitter.add(a.w_ag, a.CH, a.C, p.s_ag);
    splitter.add(a.w_bp, a.CH, a.C, p.s_bp);
    splitter.add(a.w_bg, a.CH, a.C, p.s_bg);
    splitter.add(a.w_g, a.C, a.C, p.s_g);
    splitter.add(a.w_z, a.C, a.CH, p.s_z);
    if (hipError_t es = splitter.launch(stream); es != hipSuccess) return es;  // no kernel may read unsplit weights
    auto proj = split_ab ? (fast ? trimul_proj_x3_f32<kXT, kPT, true, true> : trimul_proj_x3_f32<kXT, kPT, false, true>)
                         : (fast ? trimul_proj_x3_f32<kXT, kPT, true, false> : trimul_proj_x3_f32<kXT, kPT, false, false>);
    hipError_t e = allow_lds<trimul_proj_x3_f32<kXT, kPT, false, false>>(kLdsLimit);
    if (e == hipSuccess) e = allow_lds<trimul_proj_x3_f32<kXT, kPT, true, false>>(kLdsLimit);
    if (e == hipSuccess) e = allow_lds<trimul_proj_x3_f32<kXT, kPT, false, true>>(kLdsLimit);
    if (e == hipSuccess) e = allow_lds<trimul_proj_x3_f32<kXT, kPT, true, true>>(kLdsLimit);
    if (e == hipSuccess) e = allow_lds<trimul_out_x3_f32<kXT, kPT, false, false>>(kLdsLimit);
    if (e == hipSuccess) e = allow_lds<trimul_out_x3_f32<kXT, kPT, true, false>>(kLdsLimit);
    if (e == hipSuccess) e = allow_lds<trimul_out_x3_f32<kXT, kPT, false, true>>(kLdsLimit);
    if (e == hipSuccess) e = allow_lds<trimul_out_x3_f32<kXT, kPT, true, true>>(kLdsLimit);
    if (e == hipSuccess) e = allow_lds<trimul_contract_x3_f32>(kLdsLimit);
    if (e != hipSuccess) return e;
    const size_t lds = tile_bytes_x3(a.C, 32 * kXT * kPT) + 32 * kXT * kPT * sizeof(float);
    const int kgroups = (a.N + 32 * kXT - 1) / (32 * kXT), row_groups = (a.N + kPT - 1) / kPT;
    hipLaunchKernelGGL(proj, dim3((unsigned)((long)a.B * row_groups * kgroups)), dim3(kThreads * kPT), lds, stream, p, kgroups);
  } else if (mm) {
    hipError_t e = allow_lds<trimul_proj_mm_f32>();
    if (e == hipSuccess) e = allow_lds<trimul_out_mm_f32>();
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(trimul_proj_mm_f32, dim3(mblocks), dim3(kThreads), tile_bytes(a.C) + kTP * sizeof(float), stream,
                       p, mgroups);
  } else {
    hipLaunchKernelGGL(trimul_proj_f32, dim3((unsigned)blocks), dim3(kThreads), 0, stream, p, groups);
  }
  // the contraction has no shape or alignment condition of its own; the FMA kernel stays with the
  // FMA passes so that odd shapes run one family of kernels
  if (split_ab) {
    const int tiles_m = (a.N + kCtM - 1) / kCtM, tiles_n = (a.N + kCtN - 1) / kCtN;
    const long total = (long)a.B * a.CH * tiles_m * tiles_n;
    if (total > 0x7fffffffL - 8) return hipErrorInvalidValue;
    const int per_xcd = (int)((total + 7) / 8);
    hipLaunchKernelGGL(trimul_contract_x3_f32, dim3(per_xcd * 8), dim3(512), kContractX3Lds, stream, p, tiles_m, tiles_n,
                       (int)total, per_xcd);
  } else if (mm || x3) {
    const unsigned t = (unsigned)((a.N + 127) / 128);
    hipLaunchKernelGGL(trimul_contract_mm_f32, dim3(t, t, (unsigned)(a.B * a.CH)), dim3(kThreads), 0, stream, p.a, p.b,
                       p.x, a.N);
  } else {
    const unsigned t = (unsigned)((a.N + 63) / 64);
    hipLaunchKernelGGL(trimul_contract_f32, dim3(t, t, (unsigned)(a.B * a.CH)), dim3(kThreads), 0, stream, p.a, p.b,
                       p.x, a.N);
  }
  if (x3) {
    const size_t lds = tile_bytes_x3(a.C > a.CH ? a.C : a.CH, 32 * kXT * kPT) + 2 * kThreads * kPT * sizeof(float);
    const bool wide = a.C > 128 || a.CH > 128;
    auto kern = wide ? (fast ? trimul_out_x3_f32<kXT, kPT, true, true> : trimul_out_x3_f32<kXT, kPT, true, false>)
                     : (fast ? trimul_out_x3_f32<kXT, kPT, false, true> : trimul_out_x3_f32<kXT, kPT, false, false>);
    hipLaunchKernelGGL(kern, dim3(xblocks), dim3(kThreads * kPT), lds, stream, p, xgroups);
  }
  else if (mm)
    hipLaunchKernelGGL(trimul_out_mm_f32, dim3(mblocks), dim3(kThreads), tile_bytes(a.C) + 2 * tile_bytes(a.CH), stream,
                       p, mgroups);
  else
    hipLaunchKernelGGL(trimul_out_f32, dim3((unsigned)blocks), dim3(kThreads), 0, stream, p, groups);
  return hipGetLastError();
}

hipError_t triattn_fwd_f32(const TriattnF32Args& a, hipStream_t stream) {
  TriattnF32 p;
  p.x = a.x;
  p.mask = a.mask;
  p.xv = a.x_view;
  p.mv = a.mask_view;
  p.ln_w = a.ln_w;
  p.ln_b = a.ln_b;
  p.w_q = a.w_q;
  p.w_k = a.w_k;
  p.w_v = a.w_v;
  p.w_b = a.w_b;
  p.w_g = a.w_g;
  p.w_o = a.w_o;
  p.q = a.q;
  p.k = a.k;
  p.v = a.v;
  p.tb = a.tb;
  p.o = a.o;
  p.out = a.out;
  p.B = a.B;
  p.N = a.N;
  p.C = a.C;
  p.H = a.H;
  p.D = a.D;
  p.add_residual = a.add_residual;
  p.inf = a.inf;
  const int groups = (a.N + kP - 1) / kP;
  const long blocks = (long)a.B * a.N * groups;
  const int qgroups = (a.N + 127) / 128;
  const long cblocks = (long)a.B * a.N * a.H * qgroups;
  if (a.C > kMaxC || a.H * a.D > kMaxC || blocks > 0x7fffffffL || cblocks > 0x7fffffffL) return hipErrorInvalidValue;
  const bool mm = a.C % 8 == 0 && (a.H * a.D) % 8 == 0 && aligned16({a.w_q, a.w_k, a.w_v, a.w_b, a.w_g, a.w_o});
  const int mgroups = (a.N + kTP - 1) / kTP;
  const unsigned mblocks = (unsigned)((long)a.B * a.N * mgroups);
  const bool x3 = a.C % 16 == 0 && (a.H * a.D) % 16 == 0 && a.wsplit && aligned16({a.wsplit});
  const bool fast = a.C % 64 == 0 && (a.H * a.D) % 64 == 0 && (reinterpret_cast<uintptr_t>(a.x) & 7u) == 0 &&
                    even_strides(a.x_view);
  // head width 32 or 16 (then an even number of heads: a 32-channel tile of the projections is two of
  // them): q, k and v leave the projection pass as split operands of the split-operand core
  p.Jp = (a.N + 31) / 32 * 32;
  // (the core addresses the bias of one (batch, head) with 32-bit byte offsets)
  const bool core_x3 = x3 && (a.D == 32 || (a.D == 16 && a.H % 2 == 0)) && a.qkv_split && aligned16({a.qkv_split}) &&
                       (long)a.N * p.Jp * 4 <= 0x7fffffffL;
  p.qk_plane = (long)a.B * a.N * a.H * p.Jp * a.D;
  p.v_plane = (long)a.B * a.N * a.H * p.Jp * 32;
  p.qs = static_cast<bf16_t*>(a.qkv_split);
  p.ks = p.qs + 3 * p.qk_plane;
  p.vs = p.qs + 6 * p.qk_plane;
  const int xgroups = (a.N + 32 * kXT * kPT - 1) / (32 * kXT * kPT);
  const unsigned xblocks = (unsigned)((long)a.B * a.N * xgroups);
  if (x3) {
    WeightSplitter splitter(a.wsplit);
    const int HD = a.H * a.D;
    splitter.add(a.w_q, HD, a.C, p.s_q);
    splitter.add(a.w_k, HD, a.C, p.s_k);
    splitter.add(a.w_v, HD, a.C, p.s_v);
    splitter.add(a.w_g, HD, a.C, p.s_g);
    splitter.add(a.w_o, a.C, HD, p.s_o);
    if (hipError_t es = splitter.launch(stream); es != hipSuccess) return es;  // no kernel may read unsplit weights
    auto proj = core_x3 ? (fast ? triattn_proj_x3_f32<kXT, kPT, true, true> : triattn_proj_x3_f32<kXT, kPT, true, false>)
                        : (fast ? triattn_proj_x3_f32<kXT, kPT, false, true> : triattn_proj_x3_f32<kXT, kPT, false, false>);
    hipError_t e = allow_lds<triattn_proj_x3_f32<kXT, kPT, false, false>>(kLdsLimit);
    if (e == hipSuccess) e = allow_lds<triattn_proj_x3_f32<kXT, kPT, true, false>>(kLdsLimit);
    if (e == hipSuccess) e = allow_lds<triattn_proj_x3_f32<kXT, kPT, false, true>>(kLdsLimit);
    if (e == hipSuccess) e = allow_lds<triattn_proj_x3_f32<kXT, kPT, true, true>>(kLdsLimit);
    if (e == hipSuccess) e = allow_lds<triattn_out_x3_f32<kXT, kPT, false, false>>(kLdsLimit);
    if (e == hipSuccess) e = allow_lds<triattn_out_x3_f32<kXT, kPT, true, false>>(kLdsLimit);
    if (e == hipSuccess) e = allow_lds<triattn_out_x3_f32<kXT, kPT, false, true>>(kLdsLimit);
    if (e == hipSuccess) e = allow_lds<triattn_out_x3_f32<kXT, kPT, true, true>>(kLdsLimit);
    // the cores also hold a few static bytes (the work-group vote): ask for what they use, not for the limit
    if (e == hipSuccess) e = allow_lds<triattn_core_x3_f32<1>>(kCoreX3Lds);
    if (e == hipSuccess) e = allow_lds<triattn_core_x3_f32<2>>(kCoreX3Lds);
    if (e != hipSuccess) return e;
    const size_t lds = tile_bytes_x3(a.C, 32 * kXT * kPT) + (size_t)a.H * 32 * kXT * kPT * sizeof(float);
    hipLaunchKernelGGL(proj, dim3(xblocks), dim3(kThreads * kPT), lds, stream, p, xgroups);
  } else if (mm) {
    hipError_t e = allow_lds<triattn_proj_mm_f32>();
    if (e == hipSuccess) e = allow_lds<triattn_out_mm_f32>();
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(triattn_proj_mm_f32, dim3(mblocks), dim3(kThreads), tile_bytes(a.C), stream, p, mgroups);
  } else {
    hipLaunchKernelGGL(triattn_proj_f32, dim3((unsigned)blocks), dim3(kThreads), 0, stream, p, groups);
  }
  if (core_x3) {
    const int n_qc = (a.N + 127) / 128, n_rg = (a.N + kXRows - 1) / kXRows;
    const long total = (long)n_qc * n_rg * a.B * a.H;
    if (total > 0x7fffffffL - 8) return hipErrorInvalidValue;
    const int per_xcd = (int)((total + 7) / 8);
    hipLaunchKernelGGL(a.D == 32 ? triattn_core_x3_f32<2> : triattn_core_x3_f32<1>, dim3(per_xcd * 8), dim3(512), kCoreX3Lds,
                       stream, p, n_qc, n_rg, (int)total, per_xcd);
  } else {
    // any head width up to 64, in LDS rounded up to a multiple of 8
    void (*core)(TriattnF32, int) = nullptr;
    switch ((a.D + 7) / 8) {
      case 1: core = triattn_core_f32<8>; break;
      case 2: core = triattn_core_f32<16>; break;
      case 3: core = triattn_core_f32<24>; break;
      case 4: core = triattn_core_f32<32>; break;
      case 5: core = triattn_core_f32<40>; break;
      case 6: core = triattn_core_f32<48>; break;
      case 7: core = triattn_core_f32<56>; break;
      case 8: core = triattn_core_f32<64>; break;
      default: return hipErrorInvalidValue;
    }
    hipLaunchKernelGGL(core, dim3((unsigned)cblocks), dim3(kThreads), 0, stream, p, qgroups);
  }
  if (x3) {
    const int HD = a.H * a.D;
    const size_t lds = tile_bytes_x3(a.C > HD ? a.C : HD, 32 * kXT * kPT);
    const bool wide = a.C > 128 || HD > 128;
    auto kern = wide ? (fast ? triattn_out_x3_f32<kXT, kPT, true, true> : triattn_out_x3_f32<kXT, kPT, true, false>)
                     : (fast ? triattn_out_x3_f32<kXT, kPT, false, true> : triattn_out_x3_f32<kXT, kPT, false, false>);
    hipLaunchKernelGGL(kern, dim3(xblocks), dim3(kThreads * kPT), lds, stream, p, xgroups);
  }
  else if (mm)
    hipLaunchKernelGGL(triattn_out_mm_f32, dim3(mblocks), dim3(kThreads), tile_bytes(a.C) + tile_bytes(a.H * a.D), stream,
                       p, mgroups);
  else
    hipLaunchKernelGGL(triattn_out_f32, dim3((unsigned)blocks), dim3(kThreads), 0, stream, p, groups);
  return hipGetLastError();
}

hipError_t transition_fwd_f32(const TransitionF32Args& a, hipStream_t stream) {
  if (a.C > kMaxC || a.HID > kMaxHid) return hipErrorInvalidValue;
  TransitionF32 p;
  p.x = a.x;
  p.mask = a.mask;
  p.xv = a.x_view;
  p.mv = a.mask_view;
  p.ln_w = a.ln_w;
  p.ln_b = a.ln_b;
  p.w_a = a.w_a;
  p.w_b = a.w_b;
  p.w_out = a.w_out;
  p.out = a.out;
  p.B = a.B;
  p.N = a.N;
  p.C = a.C;
  p.HID = a.HID;
  p.add_residual = a.add_residual;
  if (a.C % 16 == 0 && a.HID % kTrHC == 0 && a.wsplit && aligned16({a.wsplit})) {
    WeightSplitter splitter(a.wsplit);
    splitter.add(a.w_a, a.HID, a.C, p.s_a);
    splitter.add(a.w_b, a.HID, a.C, p.s_b);
    splitter.add(a.w_out, a.C, a.HID, p.s_out);
    if (hipError_t es = splitter.launch(stream); es != hipSuccess) return es;  // no kernel may read unsplit weights
    const bool fast = a.C % 64 == 0 && (reinterpret_cast<uintptr_t>(a.x) & 7u) == 0 && even_strides(a.x_view);
    const bool wide = a.C > 128;
    auto kern = wide ? (fast ? transition_x3_f32<true, true> : transition_x3_f32<true, false>)
                     : (fast ? transition_x3_f32<false, true> : transition_x3_f32<false, false>);
    hipError_t e = allow_lds<transition_x3_f32<false, false>>(kLdsLimit);
    if (e == hipSuccess) e = allow_lds<transition_x3_f32<false, true>>(kLdsLimit);
    if (e == hipSuccess) e = allow_lds<transition_x3_f32<true, false>>(kLdsLimit);
    if (e == hipSuccess) e = allow_lds<transition_x3_f32<true, true>>(kLdsLimit);
    if (e != hipSuccess) return e;
    const int mgroups = (a.N + kTP - 1) / kTP;
    const long mblocks = (long)a.B * a.N * mgroups;
    if (mblocks > 0x7fffffffL) return hipErrorInvalidValue;
    hipLaunchKernelGGL(kern, dim3((unsigned)mblocks), dim3(kThreads), tile_bytes_x3(a.C, kTP) + tile_bytes_x3(kTrHC, kTP),
                       stream, p, mgroups);
    return hipGetLastError();
  }
  if (a.C % 8 == 0 && a.HID % 8 == 0 && aligned16({a.w_a, a.w_b, a.w_out})) {
    // hidden slice: as wide as keeps three work-groups on a CU (about 52 KB of LDS each)
    int hchunk = (int)((52 * 1024 - tile_bytes(a.C)) / (kTP * sizeof(float))) - 4;
    hchunk = hchunk / 32 * 32;
    if (hchunk < 32) hchunk = 32;
    if (hchunk > a.HID) hchunk = (a.HID + 31) / 32 * 32;
    const size_t mm_bytes = tile_bytes(a.C) + tile_bytes(hchunk);
    hipError_t e = allow_lds<transition_mm_f32>(kLdsLimit);
    if (e != hipSuccess) return e;
    const int mgroups = (a.N + kTP - 1) / kTP;
    const long mblocks = (long)a.B * a.N * mgroups;
    if (mblocks > 0x7fffffffL) return hipErrorInvalidValue;
    hipLaunchKernelGGL(transition_mm_f32, dim3((unsigned)mblocks), dim3(kThreads), mm_bytes, stream, p, mgroups, hchunk);
    return hipGetLastError();
  }
  const int groups = (a.N + kP - 1) / kP;
  const long blocks = (long)a.B * a.N * groups;
  hipLaunchKernelGGL(transition_f32, dim3((unsigned)blocks), dim3(kThreads), 0, stream, p, groups);
  return hipGetLastError();
}

hipError_t pair_bias_fwd_f32(const PairBiasF32Args& a, hipStream_t stream) {
  if (a.C > kMaxC) return hipErrorInvalidValue;
  PairBiasF32 p;
  p.z = a.z;
  p.zv = a.z_view;
  p.ln_w = a.ln_w;
  p.ln_b = a.ln_b;
  p.w = a.w;
  p.out = a.out;
  p.B = a.B;
  p.N = a.N;
  p.C = a.C;
  p.H = a.H;
  if (a.C % 16 == 0 && a.H <= 32) {
    const bool fast = a.C % 64 == 0 && (reinterpret_cast<uintptr_t>(a.z) & 7u) == 0 && even_strides(a.z_view);
    hipError_t e = allow_lds<pair_bias_x3_f32<false>>(kLdsLimit);
    if (e == hipSuccess) e = allow_lds<pair_bias_x3_f32<true>>(kLdsLimit);
    if (e != hipSuccess) return e;
    const int mgroups = (a.N + kTP - 1) / kTP;
    const long mblocks = (long)a.B * a.N * mgroups;
    if (mblocks > 0x7fffffffL) return hipErrorInvalidValue;
    hipLaunchKernelGGL(fast ? pair_bias_x3_f32<true> : pair_bias_x3_f32<false>, dim3((unsigned)mblocks), dim3(64),
                       tile_bytes_x3(a.C, kTP) + a.C * sizeof(float), stream, p, mgroups);
    return hipGetLastError();
  }
  const int groups = (a.N + kP - 1) / kP;
  const long blocks = (long)a.B * a.N * groups;
  hipLaunchKernelGGL(pair_bias_f32, dim3((unsigned)blocks), dim3(kThreads), 0, stream, p, groups);
  return hipGetLastError();
}

}  // namespace of3

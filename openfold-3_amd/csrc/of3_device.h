// Device-side building blocks shared by the pair-stack kernels (gfx950 / CDNA4, wave64).
//
// Conventions used by every kernel in this directory
// --------------------------------------------------
// * MFMA: v_mfma_f32_32x32x16_bf16.  Operand A is the M side (32 rows), operand B the N
//   side (32 columns); lane l supplies row/column (l % 32) and the 8 consecutive k-values
//   of k-half (l / 32).  Because A and B use the same k-assignment, any consistent
//   re-labelling of k is legal; the kernels always give lane-half h, k-step s the
//   contiguous 16-byte chunk number (2*s + h) of the 32-byte k-slice.
//   The 32x32 fp32 result lives 16 values per lane: lane l holds column (l % 32) and,
//   in register v (0..15), row 8*(v/4) + 4*(l/32) + (v%4).
// * rowperm16(): if the lane that feeds A-row r loads logical row rowperm16(r), then in
//   the result lane-half h, register v holds logical row 16*h + v, i.e. every lane owns
//   16 consecutive logical rows, which makes its share of an output row contiguous.
// * Activation tiles in LDS are [position][channel] bf16, addressed in 16-byte chunks
//   with the chunk index XOR-ed by a per-position key so that both the row-wise writers
//   and the MFMA operand readers are bank-conflict free.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace of3 {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2_t;
typedef __attribute__((__vector_size__(2 * sizeof(float)))) float f32x2_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16_t;
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4_t;  // 8 bf16
typedef __attribute__((__vector_size__(2 * sizeof(uint32_t)))) uint32_t u32x2_t;  // 4 bf16

typedef uint16_t bf16_t;  // storage type of bf16 tensors at the ABI

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLnEps = 1e-5f;

__device__ __forceinline__ f32x16_t mfma_32x32x16(u32x4_t a, u32x4_t b, f32x16_t c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                 __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
}

// the 8-deep form (two registers per operand: lane l supplies row/column l % 32 and the 4 consecutive
// k-values of k-half l / 32); same matrix-pipe time as the 16-deep one
typedef __attribute__((__vector_size__(4 * sizeof(short)))) short bf16x4_bits_t;
__device__ __forceinline__ f32x16_t mfma_32x32x8(u32x2_t a, u32x2_t b, f32x16_t c) {
  return __builtin_amdgcn_mfma_f32_32x32x8bf16_1k(__builtin_bit_cast(bf16x4_bits_t, a),
                                                  __builtin_bit_cast(bf16x4_bits_t, b), c, 0, 0, 0);
}

__device__ __forceinline__ f32x16_t zero16() {
  f32x16_t z;
#pragma unroll
  for (int i = 0; i < 16; ++i) z[i] = 0.f;
  return z;
}

__host__ __device__ __forceinline__ constexpr int rowperm16(int r) {
  return 16 * ((r >> 2) & 1) + 4 * (r >> 3) + (r & 3);
}

// ---- bf16 <-> fp32 ---------------------------------------------------------------------
__device__ __forceinline__ float bf16_lo(uint32_t u) { return __uint_as_float(u << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t u) { return __uint_as_float(u & 0xffff0000u); }
__device__ __forceinline__ float bf16_to_f32(bf16_t h) { return __uint_as_float(((uint32_t)h) << 16); }

// round-to-nearest-even pack of two floats: a -> low half, b -> high half
__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
  f32x2_t f = {a, b};
  bf16x2_t h = __builtin_convertvector(f, bf16x2_t);
  return __builtin_bit_cast(uint32_t, h);
}
__device__ __forceinline__ bf16_t to_bf16(float a) { return (bf16_t)(pack_bf16(a, 0.f) & 0xffffu); }

__device__ __forceinline__ void unpack8(u32x4_t u, float (&x)[8]) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    x[2 * i] = bf16_lo(u[i]);
    x[2 * i + 1] = bf16_hi(u[i]);
  }
}
__device__ __forceinline__ u32x4_t pack8(const float (&x)[8]) {
  u32x4_t u;
#pragma unroll
  for (int i = 0; i < 4; ++i) u[i] = pack_bf16(x[2 * i], x[2 * i + 1]);
  return u;
}

// ---- elementary functions ----------------------------------------------------------------
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }
__device__ __forceinline__ float sigmoidf_fast(float x) {
  return fast_rcp(1.f + fast_exp2(-kLog2e * x));
}
// sigmoid(x) from t = -log2(e) * x, for the passes whose normalised activations feed nothing but a gate:
// they fold the factor into the LayerNorm's weight and bias, and the gate's matrix product delivers t
__device__ __forceinline__ float sigmoid_from_scaled(float t) { return fast_rcp(1.f + fast_exp2(t)); }

// all-reduce (sum) over the LPP (8 or 16) consecutive lanes that share one position, with
// DPP lane permutations (no LDS round trips): xor 1 and xor 2 inside each quad, then
// row_half_mirror (lane i <-> 7-i of each 8) and row_mirror (i <-> 15-i of each 16), which
// pair every quad / half-row with the one holding the other partial sum.
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}
template <int LPP>
__device__ __forceinline__ float group_sum(float v) {
  static_assert(LPP == 8 || LPP == 16, "8 or 16 lanes per position");
  v += dpp_move<0xB1>(v);   // quad_perm [1,0,3,2]
  v += dpp_move<0x4E>(v);   // quad_perm [2,3,0,1]
  v += dpp_move<0x141>(v);  // row_half_mirror
  if (LPP == 16) v += dpp_move<0x140>(v);  // row_mirror
  return v;
}

// ---- LayerNorm of one position spread over C/8 lanes -------------------------------------
// raw: the lane's 8 channels (bf16 packed); w, b: affine parameters of those 8 channels.
// Statistics in fp32 (two-pass, biased variance), result rounded to bf16 like the
// reference's bf16 LayerNorm output.
template <int C>
__device__ __forceinline__ u32x4_t layer_norm_chunk(u32x4_t raw, const float (&w)[8], const float (&b)[8]) {
  float x[8];
  unpack8(raw, x);
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i) s += x[i];
  s = group_sum<C / 8>(s);
  const float mean = s * (1.f / C);
  float q = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    x[i] -= mean;
    q += x[i] * x[i];
  }
  q = group_sum<C / 8>(q);
  const float rstd = __builtin_amdgcn_rsqf(q * (1.f / C) + kLnEps);
#pragma unroll
  for (int i = 0; i < 8; ++i) x[i] = x[i] * rstd * w[i] + b[i];
  return pack8(x);
}

// load the 8 affine parameters of chunk `chunk` (channels 8*chunk .. 8*chunk+7)
__device__ __forceinline__ void load_affine8(const bf16_t* __restrict__ p, int chunk, float (&out)[8]) {
  const u32x4_t u = *reinterpret_cast<const u32x4_t*>(p + 8 * chunk);
  unpack8(u, out);
}

// ---- swizzled [position][channel] LDS tile -----------------------------------------------
// NCH = 16-byte chunks per position (C/8).  KEYSHIFT selects which position bits form the
// swizzle key: key = ((pos >> KEYSHIFT) ^ (pos >> (KEYSHIFT+3))) & (NCH-1) & 7.
template <int NCH, int KEYSHIFT>
__device__ __forceinline__ int tile_slot(int pos, int chunk) {
  const int key = ((pos >> KEYSHIFT) ^ (pos >> (KEYSHIFT + 3))) & 7 & (NCH - 1);
  return pos * NCH + (chunk ^ key);
}

// ---- global -> LDS loads without registers ------------------------------------------------------
#define OF3_LDS_AS __attribute__((address_space(3)))

// raw buffer descriptor over [base, base + bytes): 32-bit offsets, no swizzling; reads beyond the
// range return zeros
__device__ __forceinline__ __amdgpu_buffer_rsrc_t buffer_rsrc(const void* base, size_t bytes) {
  const int n = bytes > 0x7fffffffu ? 0x7fffffff : (int)bytes;
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, n, 0x00020000);
}
__device__ __forceinline__ void compiler_fence() { __asm__ volatile("" ::: "memory"); }
template <int N>
__device__ __forceinline__ void wait_vmcnt() {  // vmcnt(N) only (gfx9 encoding, N < 16)
  static_assert(N >= 0 && N < 16, "low field only");
  __builtin_amdgcn_s_waitcnt(0x0F70 | N);
}

// XCD-aware block index: hardware deals consecutive workgroup ids round-robin to the 8
// XCDs; this returns a logical id such that ids [x*per, (x+1)*per) all run on XCD x, so
// that neighbouring logical ids share one L2.  Caller launches `8*per` blocks and skips
// logical ids >= total.
__device__ __forceinline__ int xcd_logical_block(int bid, int per_xcd) {
  return (bid & 7) * per_xcd + (bid >> 3);
}

}  // namespace of3

// Internal launch interface between the C-ABI layer (of3pair_api.hip) and the kernels.
// Every launcher validates nothing: the ABI layer has already checked shapes, and each
// launcher only enqueues work on `stream` and returns hipGetLastError().
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace of3 {

typedef uint16_t bf16_t;

// Pair tensor addressing shared by the position-wise kernels.  A "row" r and a position
// k along the tile axis address z[b][r][k] at  b*stride_b + r*stride_r + k*stride_k
// (elements).  Swapping stride_r/stride_k walks the transposed tensor, which is how the
// incoming update and the ending-node attention run without a physical transpose.
struct PairView {
  int64_t stride_b, stride_r, stride_k;
};

struct TrimulProjArgs {
  const bf16_t* z;
  const float* mask;  // may be null (all ones); addressed with mask_view (channel-less)
  PairView z_view, mask_view;
  const bf16_t *ln_w, *ln_b;                  // [C]
  const bf16_t *w_ap, *w_ag, *w_bp, *w_bg;    // [CH][C]
  bf16_t *a, *b;                              // [B][CH][Np/32][Np][32]  (k-panels)
  int B, N, Np;
};
hipError_t trimul_proj_launch(const TrimulProjArgs& args, int C, int CH, hipStream_t stream);

// a, b: k-panel layout [planes][Np/32][Np][32]; x: row-major [planes][Np][Np].
// nk: the k-panels that are summed over, ceil(N / 32) (the later ones hold zeros);
// variant: 1 = 256x192 output tiles, 2 = 256x128, 3 = 256x256, 4 = 384x192 on eight waves
hipError_t trimul_contract_launch(const bf16_t* a, const bf16_t* b, bf16_t* x, int planes, int Np, int nk, int variant,
                                  hipStream_t stream);

struct TrimulOutArgs {
  const bf16_t* x;  // [B][CH][Np][Np]
  const bf16_t* z;  // gate input (and residual)
  bf16_t* out;      // same addressing as z
  PairView z_view;  // canonical orientation (i, j): x is direction-agnostic
  const bf16_t *ln_in_w, *ln_in_b;    // [C]
  const bf16_t *ln_out_w, *ln_out_b;  // [CH]
  const bf16_t *w_g;                  // [C][C]
  const bf16_t *w_z;                  // [C][CH]
  int B, N, Np;
  int add_residual;
};
hipError_t trimul_out_launch(const TrimulOutArgs& args, int C, int CH, hipStream_t stream);

struct TriattnProjArgs {
  const bf16_t* x;    // pair tensor, addressed with x_view in the module's (I, J) frame
  const float* mask;  // may be null
  PairView x_view, mask_view;
  const bf16_t *ln_w, *ln_b;          // [C]
  const bf16_t *w_q, *w_k, *w_v;      // [H*D][C]
  const bf16_t *w_b;                  // [H][C]   (linear_z: triangle bias)
  bf16_t *q, *k;                      // [B][N][H][Jp][D]
  bf16_t *vt;                         // [B][N][H][Jp/32][D][32]  (panels of 32 keys)
  float *tbias;                       // [B][H][N][Jp]   (pre-multiplied by log2 e)
  float *mbias;                       // [B][N][Jp]      (log2 e * inf * (mask-1); -inf for j >= N)
  int B, N, Jp, H;
  float inf;
};
hipError_t triattn_proj_launch(const TriattnProjArgs& args, int C, int D, hipStream_t stream);

struct TriattnFlashArgs {
  const bf16_t *q, *k, *vt;
  const float *tbias, *mbias;
  bf16_t* o;  // [B][N][N][H*D]  (module frame, channel = h*D + d)
  int B, N, Jp, H;
};
hipError_t triattn_flash_launch(const TriattnFlashArgs& args, int D, hipStream_t stream);

struct TriattnOutArgs {
  const bf16_t* o;   // [B][N][N][H*D]
  const bf16_t* x;   // module input (gate input and residual), x_view addressing
  bf16_t* out;       // x_view addressing
  PairView x_view;
  const bf16_t *ln_w, *ln_b;  // [C]
  const bf16_t *w_g;          // [H*D][C]
  const bf16_t *w_o;          // [C][H*D]
  int B, N;
  int add_residual;
};
hipError_t triattn_out_launch(const TriattnOutArgs& args, int C, int HD, hipStream_t stream);

struct TransitionArgs {
  const bf16_t* x;    // pair tensor, x_view addressing
  const float* mask;  // may be null (all ones)
  PairView x_view, mask_view;
  const bf16_t *ln_w, *ln_b;  // [C]
  const bf16_t *w_a, *w_b;    // [HID][C]  (SwiGLU linear_a: the gated half, linear_b)
  const bf16_t *w_out;        // [C][HID]
  bf16_t* out;                // x_view addressing
  int B, N, HID;              // N positions per row
  int add_residual;
  int R;                      // rows per batch element (N for a pair tensor taken row by row; 1 when the
                              // caller hands a contiguous tensor over as one row of N*N positions)
};
hipError_t transition_launch(const TransitionArgs& args, int C, hipStream_t stream);

struct PairBiasArgs {
  const bf16_t* z;            // pair tensor, z_view addressing
  PairView z_view;
  const bf16_t *ln_w, *ln_b;  // [C]; ln_b may be null (LayerNorm without offset)
  const bf16_t* w;            // [H][C]
  bf16_t* out;                // [B][H][N][N] contiguous
  int B, N, H;
};
hipError_t pair_bias_launch(const PairBiasArgs& args, int C, hipStream_t stream);

// ---- template branch (template_tail.hip): closing LayerNorm of the stack, and the fused
// LayerNorm -> mean over templates -> ReLU -> linear_t tail
struct TemplateTailArgs {
  const bf16_t* t;            // [B][T][P][C_t] contiguous, P = N*N positions
  const bf16_t *ln_w, *ln_b;  // [C_t]; used when apply_ln
  const bf16_t* w;            // linear_t, [C_z][C_t]
  bf16_t* out;                // [B][P][C_z] contiguous
  long P;
  int B, T, apply_ln;
};
hipError_t template_tail_launch(const TemplateTailArgs& args, int CT, int CZ, hipStream_t stream);
hipError_t layer_norm_launch(const bf16_t* x, const bf16_t* w, const bf16_t* b, bf16_t* out, long rows, int C,
                             hipStream_t stream);

struct TemplateTailF32Args {
  const float *t, *ln_w, *ln_b, *w;
  float* out;
  long P;
  int B, T, CT, CZ, apply_ln;
};
hipError_t template_tail_fwd_f32(const TemplateTailF32Args& args, hipStream_t stream);
hipError_t layer_norm_fwd_f32(const float* x, const float* w, const float* b, float* out, long rows, int C,
                              hipStream_t stream);

// ---- single-representation attention with pair bias (single_attn.hip), bf16, c_s = H*D = 384
struct SingleAttnArgs {
  const bf16_t* a;            // [B][N][c_s]
  const bf16_t* pair_bias;    // [B][H][N][N], the pair-bias projection of z
  const float* mask;          // [B][N] or null
  const bf16_t *ln_w, *ln_b;  // layer_norm_a
  const bf16_t *wq, *bq, *wk, *wv, *wg, *wo;
  bf16_t *q, *k;              // workspace, [B][H][Np][32] (head width padded with zeros)
  bf16_t* vt;                 // workspace, [B][H][32][Np]
  bf16_t *g, *og;             // workspace, [B][N][H*D]: gate after the sigmoid, gated attention output
  bf16_t* out;                // [B][N][c_s]; may alias a
  float inf;
  int B, N, Np, H, D, add_residual;  // Np = N rounded up to a multiple of 32
};
hipError_t single_attn_launch(const SingleAttnArgs& args, hipStream_t stream);

// ---- transition of the single representation (single_transition.hip), bf16, C = 384
struct RowTransitionArgs {
  const bf16_t* x;            // [rows][384]
  const float* mask;          // [rows] or null
  const bf16_t *ln_w, *ln_b;
  const bf16_t *wa, *wb;      // [HID][384]
  const bf16_t* wout;         // [384][HID]
  bf16_t* h;                  // workspace, [rows][HID]
  bf16_t* out;                // [rows][384]; may alias x
  long rows;
  int HID, add_residual;      // HID a multiple of 384
};
hipError_t row_transition_launch(const RowTransitionArgs& args, hipStream_t stream);

// ---- fp32 versions of the single-representation kernels (single_f32.hip)
struct SingleAttnF32Args {
  const float* a;            // [B][N][C]
  const float* pair_bias;    // [B][H][N][N]
  const float* mask;         // [B][N] or null
  const float *ln_w, *ln_b, *wq, *bq, *wk, *wv, *wg, *wo;
  float *q, *k, *v, *g, *og;  // workspace, [B][N][H*D] each
  float* out;                 // [B][N][C]; may alias a
  float inf;
  int B, N, C, H, D, add_residual;
};
hipError_t single_attn_fwd_f32(const SingleAttnF32Args& args, hipStream_t stream);

struct RowTransitionF32Args {
  const float* x;
  const float* mask;
  const float *ln_w, *ln_b, *wa, *wb, *wout;
  float* out;
  long rows;
  int C, HID, add_residual;
};
hipError_t row_transition_fwd_f32(const RowTransitionF32Args& args, hipStream_t stream);

// ---- fp32 path (pair_f32.hip): whole updates, any N, C and C_hidden <= 256, head width 16/32/64
struct TrimulF32Args {
  const float* z;
  const float* mask;                 // may be null
  PairView z_view, mask_view;        // as the projection pass walks them (swapped for incoming)
  PairView z_canonical;              // (i, j) orientation of z and out
  const float *ln_in_w, *ln_in_b, *ln_out_w, *ln_out_b;
  const float *w_ap, *w_ag, *w_bp, *w_bg, *w_g, *w_z;
  float *a, *b, *x;                  // workspace, [B][CH][N][N] each
  void* wsplit;                      // workspace, trimul_wsplit_bytes(C, CH) bytes, 16-byte aligned; may be null
  void* ab_split;                    // workspace, trimul_ab_split_bytes(B, N, CH) bytes, 16-byte aligned, may
                                     // overlap a and b; may be null
  float* out;
  int B, N, C, CH, add_residual;
};
// a and b in three bf16 terms each, rows and k padded to whole 32-wide panels
inline size_t trimul_ab_split_bytes(long B, long N, long CH) {
  const long Np = (N + 31) / 32 * 32;
  return (size_t)12 * B * CH * Np * Np;
}
hipError_t trimul_fwd_f32(const TrimulF32Args& args, hipStream_t stream);
// room for the six weight matrices split into three bf16 terms each, rows padded to multiples of 32
inline long wsplit_elems(long rows, long K) { return (rows + 31) / 32 * 32 * K; }
inline size_t trimul_wsplit_bytes(long C, long CH) {
  return (size_t)6 * (4 * wsplit_elems(CH, C) + wsplit_elems(C, C) + wsplit_elems(C, CH));
}

struct TriattnF32Args {
  const float* x;
  const float* mask;                 // may be null
  PairView x_view, mask_view;        // module frame
  const float *ln_w, *ln_b, *w_q, *w_k, *w_v, *w_b, *w_g, *w_o;
  float *q, *k, *v;                  // workspace, [B][N][H][N][D] each
  float *tb;                         // workspace, [B][H][N][N rounded up to a multiple of 32]
  float *o;                          // workspace, [B][N][N][H*D]
  void* wsplit;                      // workspace, triattn_wsplit_bytes(C, H, D) bytes, 16-byte aligned; may be null
  void* qkv_split;                   // workspace, triattn_qkv_split_bytes(B, N, H, D) bytes, 16-byte aligned, may
                                     // overlap q, k, v; may be null
  float* out;
  int B, N, C, H, D, add_residual;
  float inf;
};
hipError_t triattn_fwd_f32(const TriattnF32Args& args, hipStream_t stream);
inline size_t triattn_wsplit_bytes(long C, long H, long D) {
  return (size_t)6 * (4 * wsplit_elems(H * D, C) + wsplit_elems(C, H * D));
}
// q, k and v^T in three bf16 terms each, rows padded to whole 32-position tiles; v^T operands always
// have 32 rows (head widths below 32 leave the rest zero)
inline size_t triattn_qkv_split_bytes(long B, long N, long H, long D) {
  return (size_t)6 * B * N * H * ((N + 31) / 32 * 32) * (2 * D + (D > 32 ? D : 32));
}

struct TransitionF32Args {
  const float* x;
  const float* mask;  // may be null
  PairView x_view, mask_view;
  const float *ln_w, *ln_b, *w_a, *w_b, *w_out;  // [C], [C], [HID][C], [HID][C], [C][HID]
  void* wsplit;  // workspace, transition_wsplit_bytes(C, HID) bytes, 16-byte aligned; may be null (fp32 MFMA kernel)
  float* out;
  int B, N, C, HID, add_residual;
};
// the three weight matrices split into three bf16 terms each, rows padded to multiples of 32
inline size_t transition_wsplit_bytes(long C, long HID) {
  return (size_t)6 * (2 * wsplit_elems(HID, C) + wsplit_elems(C, HID));
}
hipError_t transition_fwd_f32(const TransitionF32Args& args, hipStream_t stream);

struct PairBiasF32Args {
  const float* z;
  PairView z_view;
  const float *ln_w, *ln_b, *w;  // ln_b may be null
  float* out;                    // [B][H][N][N]
  int B, N, C, H;
};
hipError_t pair_bias_fwd_f32(const PairBiasF32Args& args, hipStream_t stream);

}  // namespace of3

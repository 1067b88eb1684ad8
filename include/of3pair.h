/* libof3pair: MI355X (gfx950) kernels for the OpenFold3 Pairformer pair stack.
 *
 * C ABI.  Every pointer is a DEVICE pointer owned by the caller (16-byte aligned), every
 * tensor is bf16 unless stated otherwise, `stream` is a hipStream_t passed as void*.
 * Calls only enqueue work on `stream`; they never allocate, free or synchronise, and keep
 * no state between calls (apart from a per-thread "last HIP error" code and launch
 * geometry cached per process).  Return value: OF3_OK or a negative of3_status.
 *
 * Reference interfaces these entry points stand in for (paths under the reference tree):
 *   openfold3/core/model/layers/triangular_multiplicative_update.py
 *       :421-503  TriangleMultiplicativeUpdate.forward          -> of3_trimul_fwd
 *       :689-741  _cueq_triangle_mult (the existing fused-kernel operator boundary:
 *                 z, mask, norm_in/out weight+bias, the gate/projection weights,
 *                 direction, returns the update)                -> of3_trimul_fwd
 *       :485-493  LayerNorm + gated a/b projections             -> of3_trimul_proj
 *       :71-97    _combine_projections                          -> of3_trimul_contract
 *       :498-501  LayerNorm_out, linear_z, gate                 -> of3_trimul_out
 *   openfold3/core/model/layers/triangular_attention.py
 *       :102-167  TriangleAttention.forward                     -> of3_triattn_fwd
 *       :131-140  LayerNorm, mask bias, triangle bias           -> of3_triattn_proj
 *   openfold3/core/model/primitives/attention.py
 *       :265-286  Attention._prep_qkv                           -> of3_triattn_proj
 *       :625-672  _cueq_triangle_attn (q,k,v [B,I,H,J,c], triangle bias, boolean mask,
 *                 scale) / :94-135 _attention                   -> of3_triattn_flash
 *       :288-302  Attention._wrap_up (gate, linear_o)           -> of3_triattn_out
 *   openfold3/core/model/layers/transition.py
 *       :225-271  SwiGLUTransition.forward (LayerNorm, SwiGLU of
 *                 openfold3/core/model/primitives/activations.py:33-61,
 *                 linear_out, mask)                             -> of3_transition_fwd (pair tensors),
 *                                                                  of3_transition_rows_fwd (single representation)
 *   openfold3/core/model/layers/attention_pair_bias.py
 *       :151-161  _prep_bias: layer_norm_z, linear_z, permute   -> of3_pair_bias_fwd
 *       :189-244  AttentionPairBias.forward of the trunk (no AdaLN): layer_norm_a, mask bias,
 *                 Attention (attention.py:265-302, :94-135)     -> of3_attn_pair_bias_fwd
 *   openfold3/core/model/latent/template_module.py
 *       :376      TemplatePairStack's closing LayerNorm
 *                 (openfold3/core/model/primitives/normalization.py:65-84) -> of3_layer_norm_fwd
 *       :462-465  TemplateEmbedderAllAtom tail: mean over the
 *                 templates, ReLU, linear_t                     -> of3_template_tail_fwd
 *   openfold3/core/model/latent/base_blocks.py
 *       :329-335  "z = z + update" after each module            -> add_residual = 1
 *       :470-478  "z = z + pair_transition(z, mask)"            -> of3_transition_fwd, add_residual = 1
 *
 * Shapes: B batch (templates are folded into B), N tokens, C = c_z, CH = c_hidden of the
 * triangle multiplication, H heads of per-head width D.  Supported: (C, CH) in
 * {(128,128), (64,64)}; H = 4 with (C, D) in {(128,32), (64,16)}; any N >= 1.
 * NP = of3_padded_n(N) = N rounded up to a multiple of 128 is the leading dimension of
 * the intermediate buffers.
 *
 * Pair tensors are addressed by element strides {stride_b, stride_i, stride_j} with a
 * channel stride of 1; strides must be multiples of 8.  A transposed view (the
 * ending-node attention of base_blocks.py:380-404, tri_att.py:126-128) is expressed by
 * swapping stride_i and stride_j, no copy is needed.  Masks are fp32 [B,N,N] with their
 * own element strides; a null mask means all ones (tmu.py:482-483, tri_att.py:120-124).
 *
 * dtype: OF3_DTYPE_BF16 selects the MFMA kernels described above.  OF3_DTYPE_F32 (the
 * reference's default inference precision) is served by of3_trimul_fwd / of3_triattn_fwd /
 * of3_transition_fwd / of3_pair_bias_fwd / of3_layer_norm_fwd / of3_template_tail_fwd /
 * of3_attn_pair_bias_fwd / of3_transition_rows_fwd only:
 * every tensor and parameter is fp32, pointers 4-byte aligned, strides any positive
 * element counts, any N, C and CH <= 256, H*D <= 256 with D <= 64; fp32-grade
 * arithmetic in the reference's order of operations.  With channel counts in multiples of
 * 16 the two triangle modules compute every fp32 product from three bf16 terms per operand
 * on the bf16 matrix instructions (six exact products, summed in fp32; the workspace holds
 * the split weights and intermediates); channel counts in multiples of 8 and the pair
 * transition use the fp32 matrix instructions, every other shape plain FMA kernels.  The
 * stage entry points are bf16 only.
 */
#ifndef OF3PAIR_H
#define OF3PAIR_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
  OF3_OK = 0,
  OF3_EINVAL = -1, /* bad shape, stride, alignment, dtype or null pointer */
  OF3_ENOSPC = -2, /* workspace too small */
  OF3_EHIP = -3,   /* HIP launch error; code via of3_last_hip_error() */
  OF3_ESTATIC = -4 /* of3_trimul_fwd_static: the problem needs more than OF3_STATIC_SCRATCH_BYTES */
} of3_status;

typedef enum { OF3_DTYPE_F32 = 0, OF3_DTYPE_BF16 = 1 } of3_dtype;

int of3_version(void);
/* HIP error code of the last OF3_EHIP on the calling thread (0 if none). */
int of3_last_hip_error(void);
const char* of3_status_string(int status);
int64_t of3_padded_n(int64_t n);

/* ---- triangle multiplicative update ------------------------------------------------ */

/* Bytes of scratch of3_trimul_fwd needs: a, b, x = 3 * B*CH*NP*NP bf16. */
int64_t of3_trimul_workspace_bytes(int64_t B, int64_t N, int64_t C, int64_t CH);
/* The same for either dtype (fp32: a, b, x = 3 * B*CH*N*N floats). */
int64_t of3_trimul_workspace_bytes_for(int dtype, int64_t B, int64_t N, int64_t C, int64_t CH);

/* a, b: gated, masked projections, channel-major in "k-panels" of 32 contracted indices:
 * shape [B][CH][NP/32][NP][32], a[b][c][k/32][i][k%32] = a_ref[b,i,k,c] (outgoing) or
 * a_ref[b,k,i,c] (incoming).  Written: the ceil(N/32) panels that hold a k < N, their entries with k >= N
 * as zeros, rows i up to N rounded up to 4; the other panels and rows are left untouched. */
int of3_trimul_proj(const void* z, const int64_t z_strides[3], const float* mask, const int64_t mask_strides[3],
                    const void* ln_in_w, const void* ln_in_b, const void* w_a_p, const void* w_a_g,
                    const void* w_b_p, const void* w_b_g, void* a, void* b, int64_t B, int64_t N, int64_t C,
                    int64_t CH, int outgoing, void* stream);

/* x[b][c][i][j] = sum_k a[b][c][i][k] * b[b][c][j][k], the sum over the ceil(N/32) panels that hold a
 * k < N (entries with k >= N in the last of them must be zero; later panels are not read); a, b in the
 * k-panel layout above, x row-major [B][CH][NP][NP], of which rows and columns below N are meaningful.
 * variant: 0 = automatic; 1 / 2 / 3 / 4 = 256x192 / 256x128 / 256x256 / 384x192 output tiles. */
int of3_trimul_contract(const void* a, const void* b, void* x, int64_t B, int64_t N, int64_t CH, int variant,
                        void* stream);

/* The tile variant (1..4) that variant = 0 selects for this shape, or OF3_EINVAL.  A pure function of
 * the shape; lets a caller that records measurements name the kernel they were taken on.  (No
 * counterpart in the reference: the choice is internal to torch's bmm there, tmu.py:71-97.) */
int of3_trimul_contract_variant(int64_t B, int64_t N, int64_t CH);

/* out = [z +] (LN_out(x) Wz^T) * sigmoid(LN_in(z) Wg^T); out uses z's strides. */
int of3_trimul_out(const void* x, const void* z, const int64_t z_strides[3], void* out, const void* ln_in_w,
                   const void* ln_in_b, const void* ln_out_w, const void* ln_out_b, const void* w_g,
                   const void* w_z, int64_t B, int64_t N, int64_t C, int64_t CH, int add_residual, void* stream);

/* The whole module: the three kernels above on `workspace`.  out may alias z only when
 * add_residual is set or the caller no longer needs z (each position is read before it is
 * written, by the same work-group). */
int of3_trimul_fwd(const void* z, const int64_t z_strides[3], const float* mask, const int64_t mask_strides[3],
                   const void* ln_in_w, const void* ln_in_b, const void* ln_out_w, const void* ln_out_b,
                   const void* w_a_p, const void* w_a_g, const void* w_b_p, const void* w_b_g, const void* w_g,
                   const void* w_z, void* out, int64_t B, int64_t N, int64_t C, int64_t CH, int outgoing,
                   int add_residual, void* workspace, int64_t workspace_bytes, int dtype, void* stream);

/* of3_trimul_fwd for callers that cannot allocate device memory or hand a workspace over (code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has no
 * counterpart in the reference.  Same arguments, results and kernels as of3_trimul_fwd, minus the
 * workspace: a, b and x live in a scratch array built into the library, OF3_STATIC_SCRATCH_BYTES
 * per GPU, which every GPU the library runs on holds until the process ends.  The call allocates
 * and frees nothing.  Problems with of3_trimul_workspace_bytes_for(dtype, B, N, C, CH) above that
 * size return OF3_ESTATIC before anything is launched: the rule is exactly
 * of3_trimul_workspace_bytes_for(dtype, B, N, C, CH) <= OF3_STATIC_SCRATCH_BYTES (bf16:
 * B*CH*NP*NP <= 2^23, e.g. B = 1, C = CH = 128, N <= 256; fp32, whose scratch also holds the operands
 * split into bf16 terms and the split weights: B = 1, C = CH = 128 fits up to N = 142).  All calls on one
 * GPU share that GPU's array: calls that overlap on one GPU (two streams, two threads) race; calls on
 * one stream are ordered.  The first call on a device looks up the array's address and the kernels'
 * launch geometry (hipGetSymbolAddress, occupancy and attribute queries), which a stream capture does
 * not allow: make one eager call per device (any size) before capturing a graph that contains this
 * entry point; every later call issues kernel launches only. */
#define OF3_STATIC_SCRATCH_BYTES (48u << 20)
int of3_trimul_fwd_static(const void* z, const int64_t z_strides[3], const float* mask,
                          const int64_t mask_strides[3], const void* ln_in_w, const void* ln_in_b, const void* ln_out_w,
                          const void* ln_out_b, const void* w_a_p, const void* w_a_g, const void* w_b_p,
                          const void* w_b_g, const void* w_g, const void* w_z, void* out, int64_t B, int64_t N,
                          int64_t C, int64_t CH, int outgoing, int add_residual, int dtype, void* stream);

/* ---- triangle attention ------------------------------------------------------------- */

/* Scratch of of3_triattn_fwd, in this order, each part 256-byte aligned:
 *   q, k  [B][N][H][NP][D] bf16      vt [B][N][H][NP/32][D][32] bf16 (v transposed, 32-key panels)
 *   tbias [B][H][N][NP] fp32         mbias [B][N][NP] fp32       o [B][N][N][H*D] bf16 */
int64_t of3_triattn_workspace_bytes(int64_t B, int64_t N, int64_t C, int64_t H, int64_t D);
/* The same for either dtype (fp32: q, k, v, o = 4 * B*N*N*H*D floats, triangle bias B*H*N*N floats). */
int64_t of3_triattn_workspace_bytes_for(int dtype, int64_t B, int64_t N, int64_t C, int64_t H, int64_t D);

/* q is pre-multiplied by log2(e)/sqrt(D); tbias and mbias by log2(e).  Columns j >= N are written as far
 * as of3_triattn_flash reads them, i.e. up to the end of the 32-key panel that holds token N-1 (mbias -inf,
 * tbias 0, k and vt finite); the rest of the padding up to NP is left as it was.  (i, j) are the module's
 * frame as given by x_strides / mask_strides. */
int of3_triattn_proj(const void* x, const int64_t x_strides[3], const float* mask, const int64_t mask_strides[3],
                     const void* ln_w, const void* ln_b, const void* w_q, const void* w_k, const void* w_v,
                     const void* w_bias, void* q, void* k, void* vt, float* tbias, float* mbias, int64_t B,
                     int64_t N, int64_t C, int64_t H, int64_t D, float inf, void* stream);

/* o[b][i][q][h*D+d] = softmax_k(q.k + mbias[i][k] + tbias[h][q][k]) v, base-2 logits. */
int of3_triattn_flash(const void* q, const void* k, const void* vt, const float* tbias, const float* mbias, void* o,
                      int64_t B, int64_t N, int64_t H, int64_t D, void* stream);

/* out = [x +] (o * sigmoid(LN(x) Wg^T)) Wo^T; out uses x's strides. */
int of3_triattn_out(const void* o, const void* x, const int64_t x_strides[3], void* out, const void* ln_w,
                    const void* ln_b, const void* w_g, const void* w_o, int64_t B, int64_t N, int64_t C, int64_t H,
                    int64_t D, int add_residual, void* stream);

int of3_triattn_fwd(const void* x, const int64_t x_strides[3], const float* mask, const int64_t mask_strides[3],
                    const void* ln_w, const void* ln_b, const void* w_bias, const void* w_q, const void* w_k,
                    const void* w_v, const void* w_g, const void* w_o, void* out, int64_t B, int64_t N, int64_t C,
                    int64_t H, int64_t D, float inf, int add_residual, void* workspace, int64_t workspace_bytes,
                    int dtype, void* stream);

/* ---- pair transition ------------------------------------------------------------------ */

/* out = [x +] ((silu(LN(x) Wa^T) * (LN(x) Wb^T)) Wout^T) * mask, position-wise; out uses x's
 * strides and may alias x (every position is read before it is written, by the same wave).
 * w_a, w_b: [HID][C] (SwiGLU linear_a, the half passed through SiLU, and linear_b);
 * w_out: [C][HID]; HID = n*C.  No bias terms (the reference's Linear(bias=False)), no
 * workspace.  bf16: C in {64, 128}, HID a multiple of 32 and >= 128, a row's extent
 * (N-1)*stride_j elements below 2^31.  fp32: C <= 256, HID <= 1024. */
int of3_transition_fwd(const void* x, const int64_t x_strides[3], const float* mask, const int64_t mask_strides[3],
                       const void* ln_w, const void* ln_b, const void* w_a, const void* w_b, const void* w_out,
                       void* out, int64_t B, int64_t N, int64_t C, int64_t HID, int add_residual, int dtype,
                       void* stream);

/* The same with a workspace (same reference lines): in fp32, with
 * of3_transition_workspace_bytes_for(dtype, B, N, C, HID) bytes (256-byte aligned) for the weights
 * split into three bf16 terms, C a multiple of 16 and HID a multiple of 128 run on the bf16 matrix
 * instructions with fp32-grade products, as the triangle modules do; other shapes, a null workspace
 * and bf16 (which needs none: 0 bytes) behave exactly like of3_transition_fwd. */
int64_t of3_transition_workspace_bytes_for(int dtype, int64_t B, int64_t N, int64_t C, int64_t HID);
int of3_transition_fwd_ws(const void* x, const int64_t x_strides[3], const float* mask, const int64_t mask_strides[3],
                          const void* ln_w, const void* ln_b, const void* w_a, const void* w_b, const void* w_out,
                          void* out, int64_t B, int64_t N, int64_t C, int64_t HID, int add_residual, void* workspace,
                          int64_t workspace_bytes, int dtype, void* stream);

/* ---- pair-bias projection ------------------------------------------------------------- */

/* out[b][h][i][j] = sum_c LN(z[b,i,j,:])[c] * w[h][c]: the pair bias the single-representation
 * attention adds to its logits (layer_norm_z, linear_z without bias, permute_final_dims(z, [2,0,1])).
 * out is contiguous [B][H][N][N] in z's dtype; ln_b may be null (a LayerNorm created without
 * offset); w is [H][C].  No workspace.  bf16: C in {64, 128}, H <= 32; fp32: C <= 256, H <= 64. */
int of3_pair_bias_fwd(const void* z, const int64_t z_strides[3], const void* ln_w, const void* ln_b, const void* w,
                      void* out, int64_t B, int64_t N, int64_t C, int64_t H, int dtype, void* stream);

/* ---- single-representation attention with pair bias ------------------------------------ */

/* out = [a +] (softmax_k(q k^T / sqrt(D) + inf*(mask[k]-1) + pair_bias[h][q][k]) v * sigmoid(an Wg^T)) Wo^T
 * with an = LayerNorm(a), q = an Wq^T + bq, k = an Wk^T, v = an Wv^T split into H heads of width D.
 * a, out: contiguous [B][N][C_s] (out may alias a); pair_bias: contiguous [B][H][N][N], what
 * of3_pair_bias_fwd returns for this module's layer_norm_z / linear_z; mask: fp32 [B][N] or null
 * (all ones); w_q, w_k, w_v, w_g: [H*D][C_s]; b_q: [H*D]; w_o: [C_s][H*D].  bf16: the AF3 trunk
 * shape, C_s = H*D = 384, D in {8, 16, 24} (16 heads of 24); fp32: C_s <= 512, H*D <= 512,
 * D <= 64.  The workspace holds q, k, v, the gate and the gated attention output
 * (of3_attn_pair_bias_workspace_bytes: bf16; ..._for: either dtype). */
int64_t of3_attn_pair_bias_workspace_bytes(int64_t B, int64_t N, int64_t C_s, int64_t H, int64_t D);
int64_t of3_attn_pair_bias_workspace_bytes_for(int dtype, int64_t B, int64_t N, int64_t C_s, int64_t H, int64_t D);
int of3_attn_pair_bias_fwd(const void* a, const void* pair_bias, const float* mask, const void* ln_w,
                           const void* ln_b, const void* w_q, const void* b_q, const void* w_k, const void* w_v,
                           const void* w_g, const void* w_o, void* out, int64_t B, int64_t N, int64_t C_s, int64_t H,
                           int64_t D, float inf, int add_residual, void* workspace, int64_t workspace_bytes,
                           int dtype, void* stream);

/* ---- transition of the single representation ------------------------------------------- */

/* The same update as of3_transition_fwd for the single representation (PairFormerBlock's
 * single_transition, pairformer.py:118-122, :203-212): x, out contiguous [rows][C] (any leading
 * dimensions flattened; out may alias x), mask fp32 [rows] or null.  bf16: C = 384, HID a
 * multiple of 384 up to 1920, the workspace holds the hidden activations [rows][HID]; fp32: C <= 512,
 * HID <= 2048, no workspace (null, 0 is accepted). */
int64_t of3_transition_rows_workspace_bytes(int64_t rows, int64_t C, int64_t HID);
int64_t of3_transition_rows_workspace_bytes_for(int dtype, int64_t rows, int64_t C, int64_t HID);
int of3_transition_rows_fwd(const void* x, const float* mask, const void* ln_w, const void* ln_b, const void* w_a,
                            const void* w_b, const void* w_out, void* out, int64_t rows, int64_t C, int64_t HID,
                            int add_residual, void* workspace, int64_t workspace_bytes, int dtype, void* stream);

/* ---- template branch: closing LayerNorm and embedder tail ------------------------------ */

/* out = LayerNorm(x) over the last dimension of a contiguous [rows][C] tensor (eps 1e-5, affine):
 * the LayerNorm that ends TemplatePairStack.forward.  out may alias x.  bf16: C in {64, 128};
 * fp32: C <= 256. */
int of3_layer_norm_fwd(const void* x, const void* ln_w, const void* ln_b, void* out, int64_t rows, int64_t C,
                       int dtype, void* stream);

/* out[b][p][:] = W . relu((1/T) * sum_t u[b][t][p][:]) with u = LayerNorm(t) when apply_ln is
 * non-zero (t is the output of the stack's last block and the closing LayerNorm is fused in) or
 * u = t (t already normalised).  t: contiguous [B][T][P][C_t], P = N*N positions; w: linear_t,
 * [C_z][C_t], no bias; out: contiguous [B][P][C_z].  The sum runs over the templates in order,
 * its bf16 value, the division by T and the linear output are rounded where the reference's
 * bf16 tensors are.  No workspace.  bf16: C_t = 64, C_z = 128; fp32: C_t <= 256. */
int of3_template_tail_fwd(const void* t, const void* ln_w, const void* ln_b, const void* w, void* out, int64_t B,
                          int64_t T, int64_t P, int64_t C_t, int64_t C_z, int apply_ln, int dtype, void* stream);

#ifdef __cplusplus
}
#endif

#endif /* OF3PAIR_H */

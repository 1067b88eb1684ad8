// C-ABI layer of libof3pair: argument validation, workspace carving, kernel sequencing.
// The contract of every entry point is stated in include/of3pair.h.
#include "../../include/of3pair.h"

#include <hip/hip_runtime.h>

#include <mutex>

#include "of3_kernels.h"
#include "of3_launch.h"

// Built-in scratch of of3_trimul_fwd_static: one copy per GPU the library runs on, held until the
// process ends.  In host code this name is only a handle for hipGetSymbolAddress; the device
// address it yields (one per device) is what kernels and copies are given.
static __device__ __align__(256) unsigned char scratch[OF3_STATIC_SCRATCH_BYTES];

namespace {

std::mutex g_scratch_mutex;
void* g_scratch_ptr[of3::kMaxDevices];  // device address of `scratch` on each device, null until looked up

// Address of the current device's copy of `scratch` (looked up on the first call on that device).
hipError_t static_scratch(void** out) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (dev < 0 || dev >= of3::kMaxDevices) return hipErrorInvalidDevice;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return e;
    if (!ptr) return hipErrorInvalidSymbol;
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return hipSuccess;
}

thread_local int g_last_hip_error = 0;

inline int fail_hip(hipError_t e) {
  g_last_hip_error = (int)e;
  return OF3_EHIP;
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
inline int64_t align256(int64_t n) { return (n + 255) & ~(int64_t)255; }
inline int64_t padded(int64_t n) { return (n + 127) / 128 * 128; }

// The kernels count positions, tiles and work-groups in 32-bit integers: every shape whose padded
// position count B * NP * NP does not fit one is refused before any launch (such a pair tensor
// would exceed the memory of the device by far).
inline bool positions_ok(int64_t B, int64_t N) {
  if (B < 1 || N < 1 || N > (1 << 20) || B > 0x7fffffffll) return false;
  const int64_t np = padded(N);
  return np * np <= 0x7fffffffll / B;
}

inline bool trimul_dims_ok(int64_t B, int64_t N, int64_t C, int64_t CH) {
  if (!positions_ok(B, N)) return false;
  return (C == 128 && CH == 128) || (C == 64 && CH == 64);
}
inline bool triattn_dims_ok(int64_t B, int64_t N, int64_t C, int64_t H, int64_t D) {
  if (!positions_ok(B, N)) return false;
  if (B * H > 65535 || (N + 3) / 4 > 65535) return false;
  return H == 4 && ((C == 128 && D == 32) || (C == 64 && D == 16));
}
inline bool strides_ok(const int64_t s[3]) {
  return s && s[0] >= 0 && s[1] > 0 && s[2] > 0 && (s[0] % 8 == 0) && (s[1] % 8 == 0) && (s[2] % 8 == 0);
}
inline bool mask_ok(const float* mask, const int64_t s[3]) {
  if (!mask) return true;
  return s && s[0] >= 0 && s[1] >= 0 && s[2] >= 0;
}

inline bool f32_trimul_dims_ok(int64_t B, int64_t N, int64_t C, int64_t CH) {
  return positions_ok(B, N) && N <= (1 << 16) && C >= 1 && C <= 256 && CH >= 1 && CH <= 256;
}
inline bool f32_triattn_dims_ok(int64_t B, int64_t N, int64_t C, int64_t H, int64_t D) {
  return positions_ok(B, N) && N <= (1 << 16) && C >= 1 && C <= 256 && H >= 1 && D >= 1 && D <= 64 && H * D <= 256;
}
inline int64_t f32_triattn_qkv_bytes(int64_t B, int64_t N, int64_t H, int64_t D) {
  const int64_t fp32 = 3 * align256(B * N * N * H * D * 4), split = align256((int64_t)of3::triattn_qkv_split_bytes(B, N, H, D));
  return fp32 > split ? fp32 : split;
}
inline int64_t f32_trimul_ab_bytes(int64_t B, int64_t N, int64_t CH) {
  const int64_t fp32 = 2 * align256(B * CH * N * N * 4), split = align256((int64_t)of3::trimul_ab_split_bytes(B, N, CH));
  return fp32 > split ? fp32 : split;
}
// the triangle bias, rows padded to whole 32-key tiles
inline int64_t f32_triattn_tb_bytes(int64_t B, int64_t N, int64_t H) { return align256(B * H * N * ((N + 31) / 32 * 32) * 4); }
inline bool f32_strides_ok(const int64_t s[3]) { return s && s[0] >= 0 && s[1] > 0 && s[2] > 0; }
inline bool aligned4(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 3u) == 0; }

inline of3::PairView view(const int64_t s[3], bool swap) {
  of3::PairView v;
  v.stride_b = s[0];
  v.stride_r = swap ? s[2] : s[1];
  v.stride_k = swap ? s[1] : s[2];
  return v;
}
inline of3::PairView mask_view(const float* mask, const int64_t s[3], bool swap) {
  of3::PairView v = {0, 0, 0};
  if (mask) v = view(s, swap);
  return v;
}

inline const of3::bf16_t* bf(const void* p) { return static_cast<const of3::bf16_t*>(p); }
inline of3::bf16_t* bf(void* p) { return static_cast<of3::bf16_t*>(p); }

// compute units of the current device (one persistent work-group of the contraction each); 256, the
// MI355X, when no device can be asked (the shape queries are also answered without a GPU)
inline int64_t current_cu_count() {
  static int cache[of3::kMaxDevices];
  int cus = 0;
  hipError_t e = of3::per_device(cache, [](int dev, int* v) { return of3::cu_count(dev, v); }, &cus);
  if (e != hipSuccess) {
    (void)hipGetLastError();  // a shape query must not leave an error behind for the next HIP call
    return 256;
  }
  return cus >= 8 ? (cus / 8) * 8 : 8;
}

inline int contract_variant_auto(int64_t planes, int64_t Np) {
  // Cheapest of the four output tile shapes for this problem on the device's compute units (256 on
  // an MI355X): rounds of persistent work-groups x padded tile area, with a small bonus for the wider
  // tiles, which move fewer operand bytes per flop.  (768: 384x192 gives every work-group
  // exactly 4 tiles and every XCD whole planes per round; 512, 1024, 2048: 256x256 divides the
  // plane without waste.)
  const int64_t cus = current_cu_count();
  const int64_t bm[4] = {256, 256, 256, 384};
  const int64_t bn[4] = {192, 128, 256, 192};
  const double eff[4] = {0.93, 0.85, 1.00, 1.00};
  int best = 1;
  double best_cost = 0;
  for (int v = 0; v < 4; ++v) {
    const int64_t tiles = planes * ((Np + bm[v] - 1) / bm[v]) * ((Np + bn[v] - 1) / bn[v]);
    const double cost = (double)((tiles + cus - 1) / cus) * (double)(bm[v] * bn[v]) / eff[v];
    if (v == 0 || cost < best_cost) {
      best = v + 1;
      best_cost = cost;
    }
  }
  return best;
}

}  // namespace

extern "C" {

int of3_version(void) { return 1; }
int of3_last_hip_error(void) { return g_last_hip_error; }

const char* of3_status_string(int status) {
  switch (status) {
    case OF3_OK:
      return "ok";
    case OF3_EINVAL:
      return "invalid argument (shape, stride, alignment, dtype or null pointer)";
    case OF3_ENOSPC:
      return "workspace too small";
    case OF3_EHIP:
      return "HIP error (see of3_last_hip_error)";
    case OF3_ESTATIC:
      return "problem needs more scratch than the library's built-in OF3_STATIC_SCRATCH_BYTES; use the entry "
             "point that takes a workspace";
    default:
      return "unknown status";
  }
}

int64_t of3_padded_n(int64_t n) { return n < 1 ? 0 : padded(n); }

int of3_trimul_contract_variant(int64_t B, int64_t N, int64_t CH) {
  if (!positions_ok(B, N) || (CH != 128 && CH != 64)) return OF3_EINVAL;
  return contract_variant_auto(B * CH, padded(N));
}

int64_t of3_trimul_workspace_bytes(int64_t B, int64_t N, int64_t C, int64_t CH) {
  if (!trimul_dims_ok(B, N, C, CH)) return OF3_EINVAL;
  const int64_t Np = padded(N);
  return 3 * align256(B * CH * Np * Np * 2);
}

int64_t of3_trimul_workspace_bytes_for(int dtype, int64_t B, int64_t N, int64_t C, int64_t CH) {
  if (dtype == OF3_DTYPE_BF16) return of3_trimul_workspace_bytes(B, N, C, CH);
  if (dtype != OF3_DTYPE_F32 || !f32_trimul_dims_ok(B, N, C, CH)) return OF3_EINVAL;
  // a, b (fp32, or split into three bf16 terms in whole 32-wide panels), x and the weights split into three bf16 terms
  return f32_trimul_ab_bytes(B, N, CH) + align256(B * CH * N * N * 4) + align256((int64_t)of3::trimul_wsplit_bytes(C, CH));
}

int of3_trimul_proj(const void* z, const int64_t z_strides[3], const float* mask, const int64_t mask_strides[3],
                    const void* ln_in_w, const void* ln_in_b, const void* w_a_p, const void* w_a_g,
                    const void* w_b_p, const void* w_b_g, void* a, void* b, int64_t B, int64_t N, int64_t C,
                    int64_t CH, int outgoing, void* stream) {
  if (!trimul_dims_ok(B, N, C, CH) || !strides_ok(z_strides) || !mask_ok(mask, mask_strides)) return OF3_EINVAL;
  const void* ptrs[] = {z, ln_in_w, ln_in_b, w_a_p, w_a_g, w_b_p, w_b_g, a, b};
  for (const void* p : ptrs)
    if (!p || !aligned16(p)) return OF3_EINVAL;
  of3::TrimulProjArgs args;
  args.z = bf(z);
  args.mask = mask;
  args.z_view = view(z_strides, !outgoing);
  args.mask_view = mask_view(mask, mask_strides, !outgoing);
  args.ln_w = bf(ln_in_w);
  args.ln_b = bf(ln_in_b);
  args.w_ap = bf(w_a_p);
  args.w_ag = bf(w_a_g);
  args.w_bp = bf(w_b_p);
  args.w_bg = bf(w_b_g);
  args.a = bf(a);
  args.b = bf(b);
  args.B = (int)B;
  args.N = (int)N;
  args.Np = (int)padded(N);
  hipError_t e = of3::trimul_proj_launch(args, (int)C, (int)CH, static_cast<hipStream_t>(stream));
  return e == hipSuccess ? OF3_OK : fail_hip(e);
}

int of3_trimul_contract(const void* a, const void* b, void* x, int64_t B, int64_t N, int64_t CH, int variant,
                        void* stream) {
  if (!positions_ok(B, N) || (CH != 128 && CH != 64) || variant < 0 || variant > 4) return OF3_EINVAL;
  if (!a || !b || !x || !aligned16(a) || !aligned16(b) || !aligned16(x)) return OF3_EINVAL;
  const int64_t Np = padded(N);
  if (variant == 0) variant = contract_variant_auto(B * CH, Np);
  hipError_t e = of3::trimul_contract_launch(bf(a), bf(b), bf(x), (int)(B * CH), (int)Np, (int)((N + 31) / 32), variant,
                                             static_cast<hipStream_t>(stream));
  return e == hipSuccess ? OF3_OK : fail_hip(e);
}

int of3_trimul_out(const void* x, const void* z, const int64_t z_strides[3], void* out, const void* ln_in_w,
                   const void* ln_in_b, const void* ln_out_w, const void* ln_out_b, const void* w_g,
                   const void* w_z, int64_t B, int64_t N, int64_t C, int64_t CH, int add_residual, void* stream) {
  if (!trimul_dims_ok(B, N, C, CH) || !strides_ok(z_strides)) return OF3_EINVAL;
  const void* ptrs[] = {x, z, out, ln_in_w, ln_in_b, ln_out_w, ln_out_b, w_g, w_z};
  for (const void* p : ptrs)
    if (!p || !aligned16(p)) return OF3_EINVAL;
  of3::TrimulOutArgs args;
  args.x = bf(x);
  args.z = bf(z);
  args.out = bf(out);
  args.z_view = view(z_strides, false);
  args.ln_in_w = bf(ln_in_w);
  args.ln_in_b = bf(ln_in_b);
  args.ln_out_w = bf(ln_out_w);
  args.ln_out_b = bf(ln_out_b);
  args.w_g = bf(w_g);
  args.w_z = bf(w_z);
  args.B = (int)B;
  args.N = (int)N;
  args.Np = (int)padded(N);
  args.add_residual = add_residual ? 1 : 0;
  hipError_t e = of3::trimul_out_launch(args, (int)C, (int)CH, static_cast<hipStream_t>(stream));
  return e == hipSuccess ? OF3_OK : fail_hip(e);
}

int of3_trimul_fwd(const void* z, const int64_t z_strides[3], const float* mask, const int64_t mask_strides[3],
                   const void* ln_in_w, const void* ln_in_b, const void* ln_out_w, const void* ln_out_b,
                   const void* w_a_p, const void* w_a_g, const void* w_b_p, const void* w_b_g, const void* w_g,
                   const void* w_z, void* out, int64_t B, int64_t N, int64_t C, int64_t CH, int outgoing,
                   int add_residual, void* workspace, int64_t workspace_bytes, int dtype, void* stream) {
  if (dtype == OF3_DTYPE_F32) {
    if (!f32_trimul_dims_ok(B, N, C, CH) || !f32_strides_ok(z_strides) || !mask_ok(mask, mask_strides)) return OF3_EINVAL;
    const void* ptrs[] = {z, ln_in_w, ln_in_b, ln_out_w, ln_out_b, w_a_p, w_a_g, w_b_p, w_b_g, w_g, w_z, out};
    for (const void* p : ptrs)
      if (!p || !aligned4(p)) return OF3_EINVAL;
    if (!workspace || (reinterpret_cast<uintptr_t>(workspace) & 255u)) return OF3_EINVAL;
    if (workspace_bytes < of3_trimul_workspace_bytes_for(dtype, B, N, C, CH)) return OF3_ENOSPC;
    const int64_t part = align256(B * CH * N * N * 4);
    char* ws = static_cast<char*>(workspace);
    auto f = [](const void* p) { return static_cast<const float*>(p); };
    of3::TrimulF32Args a;
    a.z = f(z);
    a.mask = mask;
    a.z_view = view(z_strides, !outgoing);
    a.mask_view = mask_view(mask, mask_strides, !outgoing);
    a.z_canonical = view(z_strides, false);
    a.ln_in_w = f(ln_in_w);
    a.ln_in_b = f(ln_in_b);
    a.ln_out_w = f(ln_out_w);
    a.ln_out_b = f(ln_out_b);
    a.w_ap = f(w_a_p);
    a.w_ag = f(w_a_g);
    a.w_bp = f(w_b_p);
    a.w_bg = f(w_b_g);
    a.w_g = f(w_g);
    a.w_z = f(w_z);
    const int64_t ab = f32_trimul_ab_bytes(B, N, CH);
    a.a = reinterpret_cast<float*>(ws);
    a.b = reinterpret_cast<float*>(ws + part);
    a.ab_split = ws;  // in place of a and b
    a.x = reinterpret_cast<float*>(ws + ab);
    a.wsplit = ws + ab + part;
    a.out = static_cast<float*>(out);
    a.B = (int)B;
    a.N = (int)N;
    a.C = (int)C;
    a.CH = (int)CH;
    a.add_residual = add_residual ? 1 : 0;
    hipError_t e = of3::trimul_fwd_f32(a, static_cast<hipStream_t>(stream));
    return e == hipSuccess ? OF3_OK : (e == hipErrorInvalidValue ? (int)OF3_EINVAL : fail_hip(e));
  }
  if (dtype != OF3_DTYPE_BF16) return OF3_EINVAL;
  if (!trimul_dims_ok(B, N, C, CH)) return OF3_EINVAL;
  if (!workspace || (reinterpret_cast<uintptr_t>(workspace) & 255u)) return OF3_EINVAL;
  if (workspace_bytes < of3_trimul_workspace_bytes(B, N, C, CH)) return OF3_ENOSPC;
  const int64_t Np = padded(N);
  const int64_t part = align256(B * CH * Np * Np * 2);
  char* ws = static_cast<char*>(workspace);
  void* a = ws;
  void* b = ws + part;
  void* x = ws + 2 * part;
  int st = of3_trimul_proj(z, z_strides, mask, mask_strides, ln_in_w, ln_in_b, w_a_p, w_a_g, w_b_p, w_b_g, a, b, B, N,
                           C, CH, outgoing, stream);
  if (st != OF3_OK) return st;
  st = of3_trimul_contract(a, b, x, B, N, CH, 0, stream);
  if (st != OF3_OK) return st;
  return of3_trimul_out(x, z, z_strides, out, ln_in_w, ln_in_b, ln_out_w, ln_out_b, w_g, w_z, B, N, C, CH,
                        add_residual, stream);
}

int of3_trimul_fwd_static(const void* z, const int64_t z_strides[3], const float* mask,
                          const int64_t mask_strides[3], const void* ln_in_w, const void* ln_in_b, const void* ln_out_w,
                          const void* ln_out_b, const void* w_a_p, const void* w_a_g, const void* w_b_p,
                          const void* w_b_g, const void* w_g, const void* w_z, void* out, int64_t B, int64_t N,
                          int64_t C, int64_t CH, int outgoing, int add_residual, int dtype, void* stream) {
  const int64_t need = of3_trimul_workspace_bytes_for(dtype, B, N, C, CH);
  if (need < 0) return OF3_EINVAL;
  if (need > (int64_t)OF3_STATIC_SCRATCH_BYTES) return OF3_ESTATIC;
  void* ws = nullptr;
  hipError_t e = static_scratch(&ws);
  if (e != hipSuccess) return fail_hip(e);
  // a, b and x are written in full before they are read (entries beyond N that the kernels read
  // feed only outputs beyond N, which nothing reads), so what the last call left needs no clearing
  return of3_trimul_fwd(z, z_strides, mask, mask_strides, ln_in_w, ln_in_b, ln_out_w, ln_out_b, w_a_p, w_a_g, w_b_p,
                        w_b_g, w_g, w_z, out, B, N, C, CH, outgoing, add_residual, ws, (int64_t)OF3_STATIC_SCRATCH_BYTES,
                        dtype, stream);
}

int64_t of3_triattn_workspace_bytes(int64_t B, int64_t N, int64_t C, int64_t H, int64_t D) {
  if (!triattn_dims_ok(B, N, C, H, D)) return OF3_EINVAL;
  const int64_t Np = padded(N);
  const int64_t qkv = align256(B * N * H * Np * D * 2);
  return 3 * qkv + align256(B * H * N * Np * 4) + align256(B * N * Np * 4) + align256(B * N * N * H * D * 2);
}

int64_t of3_triattn_workspace_bytes_for(int dtype, int64_t B, int64_t N, int64_t C, int64_t H, int64_t D) {
  if (dtype == OF3_DTYPE_BF16) return of3_triattn_workspace_bytes(B, N, C, H, D);
  if (dtype != OF3_DTYPE_F32 || !f32_triattn_dims_ok(B, N, C, H, D)) return OF3_EINVAL;
  // q, k, v (fp32, or split into three bf16 terms in whole 32-position tiles), o, the triangle bias
  // and the weights split into three bf16 terms
  return f32_triattn_qkv_bytes(B, N, H, D) + align256(B * N * N * H * D * 4) + f32_triattn_tb_bytes(B, N, H) +
         align256((int64_t)of3::triattn_wsplit_bytes(C, H, D));
}

int of3_triattn_proj(const void* x, const int64_t x_strides[3], const float* mask, const int64_t mask_strides[3],
                     const void* ln_w, const void* ln_b, const void* w_q, const void* w_k, const void* w_v,
                     const void* w_bias, void* q, void* k, void* vt, float* tbias, float* mbias, int64_t B,
                     int64_t N, int64_t C, int64_t H, int64_t D, float inf, void* stream) {
  if (!triattn_dims_ok(B, N, C, H, D) || !strides_ok(x_strides) || !mask_ok(mask, mask_strides)) return OF3_EINVAL;
  const void* ptrs[] = {x, ln_w, ln_b, w_q, w_k, w_v, w_bias, q, k, vt, tbias, mbias};
  for (const void* p : ptrs)
    if (!p || !aligned16(p)) return OF3_EINVAL;
  of3::TriattnProjArgs args;
  args.x = bf(x);
  args.mask = mask;
  args.x_view = view(x_strides, false);
  args.mask_view = mask_view(mask, mask_strides, false);
  args.ln_w = bf(ln_w);
  args.ln_b = bf(ln_b);
  args.w_q = bf(w_q);
  args.w_k = bf(w_k);
  args.w_v = bf(w_v);
  args.w_b = bf(w_bias);
  args.q = bf(q);
  args.k = bf(k);
  args.vt = bf(vt);
  args.tbias = tbias;
  args.mbias = mbias;
  args.B = (int)B;
  args.N = (int)N;
  args.Jp = (int)padded(N);
  args.H = (int)H;
  args.inf = inf;
  hipError_t e = of3::triattn_proj_launch(args, (int)C, (int)D, static_cast<hipStream_t>(stream));
  return e == hipSuccess ? OF3_OK : fail_hip(e);
}

int of3_triattn_flash(const void* q, const void* k, const void* vt, const float* tbias, const float* mbias, void* o,
                      int64_t B, int64_t N, int64_t H, int64_t D, void* stream) {
  const int64_t C = (D == 32) ? 128 : 64;
  if (!triattn_dims_ok(B, N, C, H, D)) return OF3_EINVAL;
  const void* ptrs[] = {q, k, vt, tbias, mbias, o};
  for (const void* p : ptrs)
    if (!p || !aligned16(p)) return OF3_EINVAL;
  of3::TriattnFlashArgs args;
  args.q = bf(q);
  args.k = bf(k);
  args.vt = bf(vt);
  args.tbias = tbias;
  args.mbias = mbias;
  args.o = bf(o);
  args.B = (int)B;
  args.N = (int)N;
  args.Jp = (int)padded(N);
  args.H = (int)H;
  hipError_t e = of3::triattn_flash_launch(args, (int)D, static_cast<hipStream_t>(stream));
  return e == hipSuccess ? OF3_OK : fail_hip(e);
}

int of3_triattn_out(const void* o, const void* x, const int64_t x_strides[3], void* out, const void* ln_w,
                    const void* ln_b, const void* w_g, const void* w_o, int64_t B, int64_t N, int64_t C, int64_t H,
                    int64_t D, int add_residual, void* stream) {
  if (!triattn_dims_ok(B, N, C, H, D) || !strides_ok(x_strides)) return OF3_EINVAL;
  const void* ptrs[] = {o, x, out, ln_w, ln_b, w_g, w_o};
  for (const void* p : ptrs)
    if (!p || !aligned16(p)) return OF3_EINVAL;
  of3::TriattnOutArgs args;
  args.o = bf(o);
  args.x = bf(x);
  args.out = bf(out);
  args.x_view = view(x_strides, false);
  args.ln_w = bf(ln_w);
  args.ln_b = bf(ln_b);
  args.w_g = bf(w_g);
  args.w_o = bf(w_o);
  args.B = (int)B;
  args.N = (int)N;
  args.add_residual = add_residual ? 1 : 0;
  hipError_t e = of3::triattn_out_launch(args, (int)C, (int)(H * D), static_cast<hipStream_t>(stream));
  return e == hipSuccess ? OF3_OK : fail_hip(e);
}

int of3_triattn_fwd(const void* x, const int64_t x_strides[3], const float* mask, const int64_t mask_strides[3],
                    const void* ln_w, const void* ln_b, const void* w_bias, const void* w_q, const void* w_k,
                    const void* w_v, const void* w_g, const void* w_o, void* out, int64_t B, int64_t N, int64_t C,
                    int64_t H, int64_t D, float inf, int add_residual, void* workspace, int64_t workspace_bytes,
                    int dtype, void* stream) {
  if (dtype == OF3_DTYPE_F32) {
    if (!f32_triattn_dims_ok(B, N, C, H, D) || !f32_strides_ok(x_strides) || !mask_ok(mask, mask_strides)) return OF3_EINVAL;
    const void* ptrs[] = {x, ln_w, ln_b, w_bias, w_q, w_k, w_v, w_g, w_o, out};
    for (const void* p : ptrs)
      if (!p || !aligned4(p)) return OF3_EINVAL;
    if (!workspace || (reinterpret_cast<uintptr_t>(workspace) & 255u)) return OF3_EINVAL;
    if (workspace_bytes < of3_triattn_workspace_bytes_for(dtype, B, N, C, H, D)) return OF3_ENOSPC;
    const int64_t part = align256(B * N * N * H * D * 4);
    char* ws = static_cast<char*>(workspace);
    auto f = [](const void* p) { return static_cast<const float*>(p); };
    of3::TriattnF32Args a;
    a.x = f(x);
    a.mask = mask;
    a.x_view = view(x_strides, false);
    a.mask_view = mask_view(mask, mask_strides, false);
    a.ln_w = f(ln_w);
    a.ln_b = f(ln_b);
    a.w_q = f(w_q);
    a.w_k = f(w_k);
    a.w_v = f(w_v);
    a.w_b = f(w_bias);
    a.w_g = f(w_g);
    a.w_o = f(w_o);
    a.q = reinterpret_cast<float*>(ws);
    a.k = reinterpret_cast<float*>(ws + part);
    a.v = reinterpret_cast<float*>(ws + 2 * part);
    const int64_t qkv = f32_triattn_qkv_bytes(B, N, H, D);
    a.qkv_split = ws;  // in place of q, k, v
    a.o = reinterpret_cast<float*>(ws + qkv);
    a.tb = reinterpret_cast<float*>(ws + qkv + part);
    a.wsplit = ws + qkv + part + f32_triattn_tb_bytes(B, N, H);
    a.out = static_cast<float*>(out);
    a.B = (int)B;
    a.N = (int)N;
    a.C = (int)C;
    a.H = (int)H;
    a.D = (int)D;
    a.add_residual = add_residual ? 1 : 0;
    a.inf = inf;
    hipError_t e = of3::triattn_fwd_f32(a, static_cast<hipStream_t>(stream));
    return e == hipSuccess ? OF3_OK : (e == hipErrorInvalidValue ? (int)OF3_EINVAL : fail_hip(e));
  }
  if (dtype != OF3_DTYPE_BF16) return OF3_EINVAL;
  if (!triattn_dims_ok(B, N, C, H, D)) return OF3_EINVAL;
  if (!workspace || (reinterpret_cast<uintptr_t>(workspace) & 255u)) return OF3_EINVAL;
  if (workspace_bytes < of3_triattn_workspace_bytes(B, N, C, H, D)) return OF3_ENOSPC;
  const int64_t Np = padded(N);
  const int64_t qkv = align256(B * N * H * Np * D * 2);
  char* ws = static_cast<char*>(workspace);
  void* q = ws;
  void* k = ws + qkv;
  void* vt = ws + 2 * qkv;
  float* tbias = reinterpret_cast<float*>(ws + 3 * qkv);
  float* mbias = reinterpret_cast<float*>(ws + 3 * qkv + align256(B * H * N * Np * 4));
  void* o = ws + 3 * qkv + align256(B * H * N * Np * 4) + align256(B * N * Np * 4);
  int st = of3_triattn_proj(x, x_strides, mask, mask_strides, ln_w, ln_b, w_q, w_k, w_v, w_bias, q, k, vt, tbias,
                            mbias, B, N, C, H, D, inf, stream);
  if (st != OF3_OK) return st;
  st = of3_triattn_flash(q, k, vt, tbias, mbias, o, B, N, H, D, stream);
  if (st != OF3_OK) return st;
  return of3_triattn_out(o, x, x_strides, out, ln_w, ln_b, w_g, w_o, B, N, C, H, D, add_residual, stream);
}

int64_t of3_transition_workspace_bytes_for(int dtype, int64_t B, int64_t N, int64_t C, int64_t HID) {
  if (dtype == OF3_DTYPE_BF16) return (B >= 1 && N >= 1) ? 0 : (int64_t)OF3_EINVAL;
  if (dtype != OF3_DTYPE_F32 || B < 1 || N < 1 || C < 1 || C > 256 || HID < 1 || HID > 1024) return OF3_EINVAL;
  return align256((int64_t)of3::transition_wsplit_bytes(C, HID));  // the weights split into three bf16 terms
}

int of3_transition_fwd(const void* x, const int64_t x_strides[3], const float* mask, const int64_t mask_strides[3],
                       const void* ln_w, const void* ln_b, const void* w_a, const void* w_b, const void* w_out,
                       void* out, int64_t B, int64_t N, int64_t C, int64_t HID, int add_residual, int dtype,
                       void* stream) {
  return of3_transition_fwd_ws(x, x_strides, mask, mask_strides, ln_w, ln_b, w_a, w_b, w_out, out, B, N, C, HID,
                               add_residual, nullptr, 0, dtype, stream);
}

int of3_transition_fwd_ws(const void* x, const int64_t x_strides[3], const float* mask, const int64_t mask_strides[3],
                          const void* ln_w, const void* ln_b, const void* w_a, const void* w_b, const void* w_out,
                          void* out, int64_t B, int64_t N, int64_t C, int64_t HID, int add_residual, void* workspace,
                          int64_t workspace_bytes, int dtype, void* stream) {
  const void* ptrs[] = {x, ln_w, ln_b, w_a, w_b, w_out, out};
  if (!positions_ok(B, N) || !mask_ok(mask, mask_strides)) return OF3_EINVAL;
  if (dtype == OF3_DTYPE_F32) {
    if (N > (1 << 16) || C < 1 || C > 256 || HID < 1 || HID > 1024 || !f32_strides_ok(x_strides)) return OF3_EINVAL;
    for (const void* p : ptrs)
      if (!p || !aligned4(p)) return OF3_EINVAL;
    auto f = [](const void* p) { return static_cast<const float*>(p); };
    of3::TransitionF32Args a;
    a.x = f(x);
    a.mask = mask;
    a.x_view = view(x_strides, false);
    a.mask_view = mask_view(mask, mask_strides, false);
    a.ln_w = f(ln_w);
    a.ln_b = f(ln_b);
    a.w_a = f(w_a);
    a.w_b = f(w_b);
    a.w_out = f(w_out);
    // with room for the split weights the split-operand kernel runs (where the shape allows)
    a.wsplit = nullptr;
    if (workspace) {
      if (reinterpret_cast<uintptr_t>(workspace) & 255u) return OF3_EINVAL;
      if (workspace_bytes < of3_transition_workspace_bytes_for(dtype, B, N, C, HID)) return OF3_ENOSPC;
      a.wsplit = workspace;
    }
    a.out = static_cast<float*>(out);
    a.B = (int)B;
    a.N = (int)N;
    a.C = (int)C;
    a.HID = (int)HID;
    a.add_residual = add_residual ? 1 : 0;
    hipError_t e = of3::transition_fwd_f32(a, static_cast<hipStream_t>(stream));
    return e == hipSuccess ? OF3_OK : fail_hip(e);
  }
  if (dtype != OF3_DTYPE_BF16) return OF3_EINVAL;
  if (!(C == 128 || C == 64) || HID < 128 || HID % 32 != 0 || HID > (1 << 16) || !strides_ok(x_strides))
    return OF3_EINVAL;
  // A tensor (and mask) whose rows follow one another without gaps is one row of N*N positions per
  // batch element: the kernel's 256-position tiles then do not stop at row ends, which matters when
  // N is not a multiple of 256.  Positions along a row are addressed with 32-bit byte offsets.
  int64_t rows = N, row_len = N;
  if (x_strides[1] == N * x_strides[2] && (!mask || mask_strides[1] == N * mask_strides[2]) &&
      (N * N - 1) * x_strides[2] * 2 + 2 * C <= 0xffffffffll &&
      (!mask || (N * N - 1) * mask_strides[2] * 4 + 4 <= 0xffffffffll)) {
    rows = 1;
    row_len = N * N;
  }
  if ((row_len - 1) * x_strides[2] * 2 + 2 * C > 0xffffffffll) return OF3_EINVAL;
  if (mask && (row_len - 1) * mask_strides[2] * 4 + 4 > 0xffffffffll) return OF3_EINVAL;
  if (B * rows * ((row_len + 255) / 256) > 0x7fffffffll) return OF3_EINVAL;
  for (const void* p : ptrs)
    if (!p || !aligned16(p)) return OF3_EINVAL;
  of3::TransitionArgs args;
  args.x = bf(x);
  args.mask = mask;
  args.x_view = view(x_strides, false);
  args.mask_view = mask_view(mask, mask_strides, false);
  args.ln_w = bf(ln_w);
  args.ln_b = bf(ln_b);
  args.w_a = bf(w_a);
  args.w_b = bf(w_b);
  args.w_out = bf(w_out);
  args.out = bf(out);
  args.B = (int)B;
  args.N = (int)row_len;
  args.R = (int)rows;
  args.HID = (int)HID;
  args.add_residual = add_residual ? 1 : 0;
  hipError_t e = of3::transition_launch(args, (int)C, static_cast<hipStream_t>(stream));
  return e == hipSuccess ? OF3_OK : fail_hip(e);
}

int of3_pair_bias_fwd(const void* z, const int64_t z_strides[3], const void* ln_w, const void* ln_b, const void* w,
                      void* out, int64_t B, int64_t N, int64_t C, int64_t H, int dtype, void* stream) {
  if (!positions_ok(B, N) || N > (1 << 16) || H < 1 || !z || !ln_w || !w || !out) return OF3_EINVAL;
  if (dtype == OF3_DTYPE_F32) {
    if (C < 1 || C > 256 || H > 64 || !f32_strides_ok(z_strides)) return OF3_EINVAL;
    if (!aligned4(z) || !aligned4(ln_w) || !aligned4(ln_b) || !aligned4(w) || !aligned4(out)) return OF3_EINVAL;
    of3::PairBiasF32Args a;
    a.z = static_cast<const float*>(z);
    a.z_view = view(z_strides, false);
    a.ln_w = static_cast<const float*>(ln_w);
    a.ln_b = static_cast<const float*>(ln_b);
    a.w = static_cast<const float*>(w);
    a.out = static_cast<float*>(out);
    a.B = (int)B;
    a.N = (int)N;
    a.C = (int)C;
    a.H = (int)H;
    hipError_t e = of3::pair_bias_fwd_f32(a, static_cast<hipStream_t>(stream));
    return e == hipSuccess ? OF3_OK : fail_hip(e);
  }
  if (dtype != OF3_DTYPE_BF16) return OF3_EINVAL;
  if (!(C == 128 || C == 64) || H > 32 || !strides_ok(z_strides)) return OF3_EINVAL;
  if (!aligned16(z) || !aligned16(ln_w) || !aligned16(ln_b) || !aligned16(w) || !aligned16(out)) return OF3_EINVAL;
  of3::PairBiasArgs a;
  a.z = bf(z);
  a.z_view = view(z_strides, false);
  a.ln_w = bf(ln_w);
  a.ln_b = bf(ln_b);
  a.w = bf(w);
  a.out = bf(out);
  a.B = (int)B;
  a.N = (int)N;
  a.H = (int)H;
  hipError_t e = of3::pair_bias_launch(a, (int)C, static_cast<hipStream_t>(stream));
  return e == hipSuccess ? OF3_OK : fail_hip(e);
}

int of3_layer_norm_fwd(const void* x, const void* ln_w, const void* ln_b, void* out, int64_t rows, int64_t C,
                       int dtype, void* stream) {
  if (rows < 1 || !x || !ln_w || !ln_b || !out) return OF3_EINVAL;
  if (dtype == OF3_DTYPE_F32) {
    if (C < 1 || C > 256) return OF3_EINVAL;
    if (!aligned4(x) || !aligned4(ln_w) || !aligned4(ln_b) || !aligned4(out)) return OF3_EINVAL;
    hipError_t e = of3::layer_norm_fwd_f32(static_cast<const float*>(x), static_cast<const float*>(ln_w),
                                           static_cast<const float*>(ln_b), static_cast<float*>(out), (long)rows,
                                           (int)C, static_cast<hipStream_t>(stream));
    return e == hipSuccess ? OF3_OK : fail_hip(e);
  }
  if (dtype != OF3_DTYPE_BF16) return OF3_EINVAL;
  if (!(C == 128 || C == 64)) return OF3_EINVAL;
  if (!aligned16(x) || !aligned16(ln_w) || !aligned16(ln_b) || !aligned16(out)) return OF3_EINVAL;
  hipError_t e = of3::layer_norm_launch(bf(x), bf(ln_w), bf(ln_b), bf(out), (long)rows, (int)C,
                                        static_cast<hipStream_t>(stream));
  return e == hipSuccess ? OF3_OK : fail_hip(e);
}

int of3_template_tail_fwd(const void* t, const void* ln_w, const void* ln_b, const void* w, void* out, int64_t B,
                          int64_t T, int64_t P, int64_t C_t, int64_t C_z, int apply_ln, int dtype, void* stream) {
  if (B < 1 || T < 1 || T > 1024 || P < 1 || !t || !w || !out) return OF3_EINVAL;
  if (apply_ln && (!ln_w || !ln_b)) return OF3_EINVAL;
  if (B > 0x7fffffffll || P > (1ll << 40)) return OF3_EINVAL;
  if (dtype == OF3_DTYPE_F32) {
    if (C_t < 1 || C_t > 256 || C_z < 1 || C_z > 4096) return OF3_EINVAL;
    if (!aligned4(t) || !aligned4(ln_w) || !aligned4(ln_b) || !aligned4(w) || !aligned4(out)) return OF3_EINVAL;
    of3::TemplateTailF32Args a;
    a.t = static_cast<const float*>(t);
    a.ln_w = static_cast<const float*>(ln_w);
    a.ln_b = static_cast<const float*>(ln_b);
    a.w = static_cast<const float*>(w);
    a.out = static_cast<float*>(out);
    a.P = (long)P;
    a.B = (int)B;
    a.T = (int)T;
    a.CT = (int)C_t;
    a.CZ = (int)C_z;
    a.apply_ln = apply_ln ? 1 : 0;
    hipError_t e = of3::template_tail_fwd_f32(a, static_cast<hipStream_t>(stream));
    return e == hipSuccess ? OF3_OK : fail_hip(e);
  }
  if (dtype != OF3_DTYPE_BF16) return OF3_EINVAL;
  if (C_t != 64 || C_z != 128) return OF3_EINVAL;
  if (!aligned16(t) || !aligned16(ln_w) || !aligned16(ln_b) || !aligned16(w) || !aligned16(out)) return OF3_EINVAL;
  of3::TemplateTailArgs a;
  a.t = bf(t);
  a.ln_w = bf(ln_w);
  a.ln_b = bf(ln_b);
  a.w = bf(w);
  a.out = bf(out);
  a.P = (long)P;
  a.B = (int)B;
  a.T = (int)T;
  a.apply_ln = apply_ln ? 1 : 0;
  hipError_t e = of3::template_tail_launch(a, (int)C_t, (int)C_z, static_cast<hipStream_t>(stream));
  return e == hipSuccess ? OF3_OK : fail_hip(e);
}

int64_t of3_attn_pair_bias_workspace_bytes(int64_t B, int64_t N, int64_t C_s, int64_t H, int64_t D) {
  if (B < 1 || N < 1 || N > (1 << 16) || C_s != 384 || H < 1 || D < 8 || D > 24 || (D % 8) != 0 || H * D != C_s)
    return OF3_EINVAL;
  const int64_t Np = (N + 31) / 32 * 32;
  return 3 * align256(B * H * Np * 32 * 2) + 2 * align256(B * N * H * D * 2);
}

int64_t of3_attn_pair_bias_workspace_bytes_for(int dtype, int64_t B, int64_t N, int64_t C_s, int64_t H, int64_t D) {
  if (dtype == OF3_DTYPE_BF16) return of3_attn_pair_bias_workspace_bytes(B, N, C_s, H, D);
  if (dtype != OF3_DTYPE_F32 || B < 1 || B > 65535 || N < 1 || N > (1 << 16) || C_s < 1 || C_s > 512 || H < 1 ||
      D < 1 || D > 64 || H * D > 512)
    return OF3_EINVAL;
  return 5 * align256(B * N * H * D * 4);
}

int of3_attn_pair_bias_fwd(const void* a, const void* pair_bias, const float* mask, const void* ln_w,
                           const void* ln_b, const void* w_q, const void* b_q, const void* w_k, const void* w_v,
                           const void* w_g, const void* w_o, void* out, int64_t B, int64_t N, int64_t C_s, int64_t H,
                           int64_t D, float inf, int add_residual, void* workspace, int64_t workspace_bytes,
                           int dtype, void* stream) {
  if (dtype == OF3_DTYPE_F32) {
    const int64_t need32 = of3_attn_pair_bias_workspace_bytes_for(dtype, B, N, C_s, H, D);
    if (need32 < 0) return OF3_EINVAL;
    const void* p32[] = {a, pair_bias, ln_w, ln_b, w_q, b_q, w_k, w_v, w_g, w_o, out, workspace};
    for (const void* p : p32)
      if (!p || !aligned4(p)) return OF3_EINVAL;
    if (mask && !aligned4(mask)) return OF3_EINVAL;
    if (workspace_bytes < need32) return OF3_ENOSPC;
    const int64_t part = align256(B * N * H * D * 4);
    char* ws = static_cast<char*>(workspace);
    auto f = [](const void* p) { return static_cast<const float*>(p); };
    of3::SingleAttnF32Args s;
    s.a = f(a);
    s.pair_bias = f(pair_bias);
    s.mask = mask;
    s.ln_w = f(ln_w);
    s.ln_b = f(ln_b);
    s.wq = f(w_q);
    s.bq = f(b_q);
    s.wk = f(w_k);
    s.wv = f(w_v);
    s.wg = f(w_g);
    s.wo = f(w_o);
    s.q = reinterpret_cast<float*>(ws);
    s.k = reinterpret_cast<float*>(ws + part);
    s.v = reinterpret_cast<float*>(ws + 2 * part);
    s.g = reinterpret_cast<float*>(ws + 3 * part);
    s.og = reinterpret_cast<float*>(ws + 4 * part);
    s.out = static_cast<float*>(out);
    s.inf = inf;
    s.B = (int)B;
    s.N = (int)N;
    s.C = (int)C_s;
    s.H = (int)H;
    s.D = (int)D;
    s.add_residual = add_residual ? 1 : 0;
    hipError_t e = of3::single_attn_fwd_f32(s, static_cast<hipStream_t>(stream));
    return e == hipSuccess ? OF3_OK : fail_hip(e);
  }
  if (dtype != OF3_DTYPE_BF16) return OF3_EINVAL;
  const int64_t need = of3_attn_pair_bias_workspace_bytes(B, N, C_s, H, D);
  if (need < 0 || B > 65535) return OF3_EINVAL;
  const void* ptrs[] = {a, pair_bias, ln_w, ln_b, w_q, b_q, w_k, w_v, w_g, w_o, out, workspace};
  for (const void* p : ptrs)
    if (!p || !aligned16(p)) return OF3_EINVAL;
  if (mask && !aligned4(mask)) return OF3_EINVAL;
  if (workspace_bytes < need) return OF3_ENOSPC;
  const int64_t Np = (N + 31) / 32 * 32;
  const int64_t qk = align256(B * H * Np * 32 * 2), go = align256(B * N * H * D * 2);
  char* ws = static_cast<char*>(workspace);
  of3::SingleAttnArgs s;
  s.a = bf(a);
  s.pair_bias = bf(pair_bias);
  s.mask = mask;
  s.ln_w = bf(ln_w);
  s.ln_b = bf(ln_b);
  s.wq = bf(w_q);
  s.bq = bf(b_q);
  s.wk = bf(w_k);
  s.wv = bf(w_v);
  s.wg = bf(w_g);
  s.wo = bf(w_o);
  s.q = reinterpret_cast<of3::bf16_t*>(ws);
  s.k = reinterpret_cast<of3::bf16_t*>(ws + qk);
  s.vt = reinterpret_cast<of3::bf16_t*>(ws + 2 * qk);
  s.g = reinterpret_cast<of3::bf16_t*>(ws + 3 * qk);
  s.og = reinterpret_cast<of3::bf16_t*>(ws + 3 * qk + go);
  s.out = bf(out);
  s.inf = inf;
  s.B = (int)B;
  s.N = (int)N;
  s.Np = (int)Np;
  s.H = (int)H;
  s.D = (int)D;
  s.add_residual = add_residual ? 1 : 0;
  hipError_t e = of3::single_attn_launch(s, static_cast<hipStream_t>(stream));
  return e == hipSuccess ? OF3_OK : fail_hip(e);
}

int64_t of3_transition_rows_workspace_bytes(int64_t rows, int64_t C, int64_t HID) {
  if (rows < 1 || rows > (1ll << 31) || C != 384 || HID < C || (HID % C) != 0 || HID > 5 * C) return OF3_EINVAL;
  return align256(rows * HID * 2);
}

int64_t of3_transition_rows_workspace_bytes_for(int dtype, int64_t rows, int64_t C, int64_t HID) {
  if (dtype == OF3_DTYPE_BF16) return of3_transition_rows_workspace_bytes(rows, C, HID);
  if (dtype != OF3_DTYPE_F32 || rows < 1 || rows > (1ll << 31) || C < 1 || C > 512 || HID < 1 || HID > 2048)
    return OF3_EINVAL;
  return 0;  // the hidden activations stay on chip
}

int of3_transition_rows_fwd(const void* x, const float* mask, const void* ln_w, const void* ln_b, const void* w_a,
                            const void* w_b, const void* w_out, void* out, int64_t rows, int64_t C, int64_t HID,
                            int add_residual, void* workspace, int64_t workspace_bytes, int dtype, void* stream) {
  if (dtype == OF3_DTYPE_F32) {
    if (of3_transition_rows_workspace_bytes_for(dtype, rows, C, HID) < 0) return OF3_EINVAL;
    const void* p32[] = {x, ln_w, ln_b, w_a, w_b, w_out, out};
    for (const void* p : p32)
      if (!p || !aligned4(p)) return OF3_EINVAL;
    if (mask && !aligned4(mask)) return OF3_EINVAL;
    auto f = [](const void* p) { return static_cast<const float*>(p); };
    of3::RowTransitionF32Args a;
    a.x = f(x);
    a.mask = mask;
    a.ln_w = f(ln_w);
    a.ln_b = f(ln_b);
    a.wa = f(w_a);
    a.wb = f(w_b);
    a.wout = f(w_out);
    a.out = static_cast<float*>(out);
    a.rows = (long)rows;
    a.C = (int)C;
    a.HID = (int)HID;
    a.add_residual = add_residual ? 1 : 0;
    hipError_t e = of3::row_transition_fwd_f32(a, static_cast<hipStream_t>(stream));
    return e == hipSuccess ? OF3_OK : fail_hip(e);
  }
  if (dtype != OF3_DTYPE_BF16) return OF3_EINVAL;
  const int64_t need = of3_transition_rows_workspace_bytes(rows, C, HID);
  if (need < 0) return OF3_EINVAL;
  const void* ptrs[] = {x, ln_w, ln_b, w_a, w_b, w_out, out, workspace};
  for (const void* p : ptrs)
    if (!p || !aligned16(p)) return OF3_EINVAL;
  if (mask && !aligned4(mask)) return OF3_EINVAL;
  if (workspace_bytes < need) return OF3_ENOSPC;
  of3::RowTransitionArgs a;
  a.x = bf(x);
  a.mask = mask;
  a.ln_w = bf(ln_w);
  a.ln_b = bf(ln_b);
  a.wa = bf(w_a);
  a.wb = bf(w_b);
  a.wout = bf(w_out);
  a.h = static_cast<of3::bf16_t*>(workspace);
  a.out = bf(out);
  a.rows = (long)rows;
  a.HID = (int)HID;
  a.add_residual = add_residual ? 1 : 0;
  hipError_t e = of3::row_transition_launch(a, static_cast<hipStream_t>(stream));
  return e == hipSuccess ? OF3_OK : fail_hip(e);
}

}  // extern "C"

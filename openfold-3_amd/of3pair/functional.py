"""Tensor-level wrappers over the C ABI: the functional boundary the reference already has
for alternative kernels (_cueq_triangle_mult, tmu.py:689-741; Attention's kernel branch,
attention.py:366-413), here with a single implementation and no dispatch.

All functions run on the current CUDA(HIP) stream of the tensors' device, are forward-only
and accept bf16 or fp32 pair tensors shaped [*, N, N, C] (any number of leading batch
dimensions, a transposed view in the two N dimensions is fine and is not copied).  bf16 runs
the bf16 MFMA kernels (built for the AF3 widths; any other width runs on the fp32 kernels and is
rounded to bf16 at the end); fp32 (the reference's default inference precision) runs the library's
fp32 kernels (slower, the precision path); parameters are converted to the tensor's dtype.
"""
from __future__ import annotations

import torch

from . import _lib

_workspaces: dict = {}
_in_graph: set = set()  # keys of the buffers a stream capture has handed to kernels
_retired: list = []


def _workspace(device, nbytes: int) -> torch.Tensor:
    """Grow-only scratch per (device, current stream), owned by this Python layer (the library
    allocates nothing).  Kernels on one stream are ordered, so all modules running on a stream share
    its buffer; another stream gets a buffer of its own.  A buffer that is outgrown is freed, unless a
    stream capture has used it: a HIP graph captured earlier still replays kernels that point into it
    and the caching allocator must not hand that memory to another tensor, so such a buffer is kept
    alive until release_workspaces()."""
    key = (device, torch.cuda.current_stream(device).cuda_stream)
    capturing = torch.cuda.is_current_stream_capturing()
    buf = _workspaces.get(key)
    if buf is None or buf.numel() < nbytes:
        if buf is not None and key in _in_graph:
            _retired.append(buf)
        _in_graph.discard(key)
        # an eager buffer goes back to the allocator before its successor is requested (kernels already
        # queued on this stream keep it valid: the allocator reuses it for later work of the stream only)
        _workspaces.pop(key, None)
        del buf
        buf = torch.empty(int(nbytes), dtype=torch.uint8, device=device)
        _workspaces[key] = buf
    if capturing:
        _in_graph.add(key)
    return buf


def release_workspaces():
    """Drops every scratch buffer, current and outgrown.  Only when no captured graph that used them
    will be replayed again."""
    _workspaces.clear()
    _in_graph.clear()
    _retired.clear()


def _require_gpu(t: torch.Tensor, name: str) -> int:
    """Returns the library's dtype code of t."""
    if not t.is_cuda:
        raise RuntimeError("%s must live on the GPU: the pair-stack kernels have no CPU path" % name)
    if t.dtype == torch.bfloat16:
        return _lib.OF3_DTYPE_BF16
    if t.dtype == torch.float32:
        return _lib.OF3_DTYPE_F32
    raise ValueError("%s must be bfloat16 or float32 (got %s)" % (name, t.dtype))


def _through_fp32(fn, x, inplace, *args, **kwargs):
    """A bf16 call whose channel widths the bf16 MFMA kernels do not serve (they are built for the
    AF3 widths) runs on the library's fp32 kernels instead: the activations are widened on the
    device, every operation is the fp32 one, the result is rounded to bf16 once at the end.  Still
    the HIP path; slower, and closer to an fp32 evaluation than the reference's bf16 path is."""
    out = fn(x.float(), *args, inplace=False, **kwargs).to(torch.bfloat16)
    if inplace:
        x.copy_(out)
        return x
    return out


def _flatten_pair(z: torch.Tensor):
    """[*, N, N, C] -> a 4-D view [B, N, N, C] with unit channel stride, no copy when the
    leading dimensions can be merged."""
    if z.dim() < 3:
        raise ValueError("pair tensor must be [*, N, N, C]")
    n1, n2, c = z.shape[-3:]
    if n1 != n2:
        raise ValueError("pair tensor must be square in its two token dimensions, got %s" % (tuple(z.shape),))
    if z.stride(-1) != 1 and c != 1:
        z = z.contiguous()
    lead = z.shape[:-3]
    if len(lead) == 0:
        z4 = z.unsqueeze(0)
    elif len(lead) == 1:
        z4 = z
    else:
        try:
            z4 = z.view(-1, n1, n2, c)
        except RuntimeError:
            z4 = z.reshape(-1, n1, n2, c)
    if z.dtype == torch.bfloat16 and (any(s % 8 for s in z4.stride()[:3]) or z4.data_ptr() % 16):
        z4 = z4.contiguous()
    return z4, lead


def _mask_arg(mask, lead, B, N, device):
    if mask is None:
        return None, None, None
    m = mask
    if m.shape[-2:] != (N, N):
        raise ValueError("mask must be [*, N, N]")
    if m.dtype != torch.float32:
        m = m.to(torch.float32)
    m = m.expand(*lead, N, N) if len(lead) else m
    m3 = m.reshape(B, N, N) if m.dim() != 3 else m
    return m3, m3.data_ptr(), _lib.strides3(m3.stride())


def _w(t: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """Parameter as a contiguous device tensor of the activations' dtype (what a module cast
    with .to(dtype) already holds; otherwise converted once per call)."""
    if t.dtype != dtype or not t.is_contiguous():
        t = t.detach().to(dtype).contiguous()
    return t


def _stream(t: torch.Tensor):
    return torch.cuda.current_stream(t.device).cuda_stream


def _out_like(z4: torch.Tensor) -> torch.Tensor:
    return torch.empty_strided(z4.shape, z4.stride(), dtype=z4.dtype, device=z4.device)


def _finish(z, z4, out4, lead, inplace):
    out = out4.view(z.shape)
    if not inplace:
        return out
    if z4.data_ptr() != z.data_ptr():  # the kernels ran on a re-laid-out copy
        z.copy_(out)
    return z


def triangle_multiplicative_update(z, mask, norm_in_weight, norm_in_bias, norm_out_weight, norm_out_bias,
                                   a_p_weight, a_g_weight, b_p_weight, b_g_weight, g_out_weight, p_out_weight,
                                   outgoing: bool, add_residual: bool = False, inplace: bool = False):
    """Update of tmu.py:482-503, or z + update when add_residual.  With inplace the result
    overwrites z (the reference's inplace_safe contract, tmu.py:154-173)."""
    code = _require_gpu(z, "z")
    lib = _lib.load()
    z4, lead = _flatten_pair(z)
    B, N, _, C = z4.shape
    CH = a_p_weight.shape[0]
    nbytes = lib.of3_trimul_workspace_bytes_for(code, B, N, C, CH)
    if nbytes < 0 and code == _lib.OF3_DTYPE_BF16 and lib.of3_trimul_workspace_bytes_for(_lib.OF3_DTYPE_F32, B, N, C, CH) >= 0:
        return _through_fp32(triangle_multiplicative_update, z, inplace, mask, norm_in_weight, norm_in_bias,
                             norm_out_weight, norm_out_bias, a_p_weight, a_g_weight, b_p_weight, b_g_weight,
                             g_out_weight, p_out_weight, outgoing=outgoing, add_residual=add_residual)
    if nbytes < 0:
        raise ValueError("triangle multiplication: bf16 supports (c_z, c_hidden) = (128,128) or (64,64), fp32 any "
                         "widths up to 256; got (%d,%d) in %s" % (C, CH, z.dtype))
    keep = [_w(t, z.dtype) for t in (norm_in_weight, norm_in_bias, norm_out_weight, norm_out_bias, a_p_weight, a_g_weight,
                            b_p_weight, b_g_weight, g_out_weight, p_out_weight)]
    m3, mptr, mstr = _mask_arg(mask, lead, B, N, z.device)
    out4 = z4 if inplace else _out_like(z4)
    ws = _workspace(z.device, nbytes)
    with torch.cuda.device(z.device):
        st = lib.of3_trimul_fwd(z4.data_ptr(), _lib.strides3(z4.stride()[:3]), mptr, mstr, *[k.data_ptr() for k in keep],
                                out4.data_ptr(), B, N, C, CH, int(bool(outgoing)), int(bool(add_residual)),
                                ws.data_ptr(), ws.numel(), code, _stream(z))
    _lib.check(st, "of3_trimul_fwd")
    return _finish(z, z4, out4, lead, inplace)


def triangle_attention(x, mask, norm_weight, norm_bias, bias_weight, q_weight, k_weight, v_weight, g_weight,
                       o_weight, no_heads: int, inf: float = 1e9, add_residual: bool = False,
                       inplace: bool = False):
    """Update of tri_att.py:102-167 for a starting-node module; hand in the transposed view
    for the ending node (base_blocks.py:380-404 does exactly that)."""
    code = _require_gpu(x, "x")
    lib = _lib.load()
    x4, lead = _flatten_pair(x)
    B, N, _, C = x4.shape
    H = int(no_heads)
    D = q_weight.shape[0] // H
    nbytes = lib.of3_triattn_workspace_bytes_for(code, B, N, C, H, D)
    if nbytes < 0 and code == _lib.OF3_DTYPE_BF16 and lib.of3_triattn_workspace_bytes_for(_lib.OF3_DTYPE_F32, B, N, C, H, D) >= 0:
        return _through_fp32(triangle_attention, x, inplace, mask, norm_weight, norm_bias, bias_weight, q_weight,
                             k_weight, v_weight, g_weight, o_weight, no_heads=no_heads, inf=inf,
                             add_residual=add_residual)
    if nbytes < 0:
        raise ValueError("triangle attention: bf16 supports 4 heads with (c_in, c_head) = (128,32) or (64,16), fp32 "
                         "c_in <= 256, head widths up to 64 and heads * c_head <= 256; got c_in=%d heads=%d c_head=%d in %s" % (C, H, D, x.dtype))
    keep = [_w(t, x.dtype) for t in (norm_weight, norm_bias, bias_weight, q_weight, k_weight, v_weight, g_weight, o_weight)]
    m3, mptr, mstr = _mask_arg(mask, lead, B, N, x.device)
    out4 = x4 if inplace else _out_like(x4)
    ws = _workspace(x.device, nbytes)
    with torch.cuda.device(x.device):
        st = lib.of3_triattn_fwd(x4.data_ptr(), _lib.strides3(x4.stride()[:3]), mptr, mstr,
                                 *[k.data_ptr() for k in keep], out4.data_ptr(), B, N, C, H, D, float(inf),
                                 int(bool(add_residual)), ws.data_ptr(), ws.numel(), code, _stream(x))
    _lib.check(st, "of3_triattn_fwd")
    return _finish(x, x4, out4, lead, inplace)


def swiglu_transition(x, mask, norm_weight, norm_bias, a_weight, b_weight, out_weight, add_residual: bool = False,
                      inplace: bool = False):
    """Update of transition.py:256-268 (LayerNorm, SwiGLU, linear_out, mask), or x + update when
    add_residual.  x [*, N, N, C], mask [*, N, N] or None; a_weight / b_weight [n*C, C] are
    SwiGLU's linear_a (through SiLU) and linear_b, out_weight [C, n*C].  With C = 384 (the single
    representation) x is [*, 384] and mask [*]: any leading dimensions (the transition is
    position-wise, so a pair tensor of 384 channels takes that route too and gets the same result).
    A tensor of fewer than three dimensions cannot be a pair tensor and is taken as rows [*, C] too."""
    code = _require_gpu(x, "x")
    lib = _lib.load()
    if x.shape[-1] == 384 or x.dim() < 3:  # the single representation: position-wise over [*, C] rows
        return _swiglu_transition_rows(x, mask, norm_weight, norm_bias, a_weight, b_weight, out_weight,
                                       add_residual, inplace, code)
    x4, lead = _flatten_pair(x)
    B, N, _, C = x4.shape
    HID = a_weight.shape[0]
    if tuple(a_weight.shape) != (HID, C) or tuple(b_weight.shape) != (HID, C) or tuple(out_weight.shape) != (C, HID):
        raise ValueError("transition weights must be [n*C, C], [n*C, C] and [C, n*C]")
    # which kernels serve these widths is decided from the shape alone: any other refusal of the
    # library (alignment, strides, null pointers) is the caller's error and is raised
    bf16_widths = C in (64, 128) and HID >= 128 and HID % 32 == 0 and HID <= (1 << 16)
    fp32_widths = 1 <= C <= 256 and 1 <= HID <= 1024
    if code == _lib.OF3_DTYPE_BF16 and not bf16_widths and fp32_widths:
        return _through_fp32(swiglu_transition, x, inplace, mask, norm_weight, norm_bias, a_weight, b_weight, out_weight,
                             add_residual=add_residual)
    served = bf16_widths if code == _lib.OF3_DTYPE_BF16 else fp32_widths
    keep = [_w(t, x.dtype) for t in (norm_weight, norm_bias, a_weight, b_weight, out_weight)]
    m3, mptr, mstr = _mask_arg(mask, lead, B, N, x.device)
    out4 = x4 if inplace else _out_like(x4)
    need = lib.of3_transition_workspace_bytes_for(code, B, N, C, HID)  # fp32: room for the split weights
    ws = _workspace(x.device, need) if need > 0 else None
    with torch.cuda.device(x.device):
        st = lib.of3_transition_fwd_ws(x4.data_ptr(), _lib.strides3(x4.stride()[:3]), mptr, mstr,
                                       *[k.data_ptr() for k in keep], out4.data_ptr(), B, N, C, HID,
                                       int(bool(add_residual)), ws.data_ptr() if ws is not None else None,
                                       need if ws is not None else 0, code, _stream(x))
    if st == _lib.OF3_EINVAL and not served:
        raise ValueError("pair transition: bf16 supports c_in 64 or 128 with a hidden width n*c_in that is a multiple "
                         "of 32 and at least 128, fp32 c_in <= 256 and n*c_in <= 1024; got c_in=%d hidden=%d in %s"
                         % (C, HID, x.dtype))
    _lib.check(st, "of3_transition_fwd")
    return _finish(x, x4, out4, lead, inplace)


def _swiglu_transition_rows(x, mask, norm_weight, norm_bias, a_weight, b_weight, out_weight, add_residual, inplace,
                            code):
    """The transition over the single representation s [*, 384] (pairformer.py:203-212): every
    leading dimension is a row; mask [*] or None."""
    lib = _lib.load()
    C = x.shape[-1]
    HID = a_weight.shape[0]
    if tuple(a_weight.shape) != (HID, C) or tuple(b_weight.shape) != (HID, C) or tuple(out_weight.shape) != (C, HID):
        raise ValueError("transition weights must be [n*C, C], [n*C, C] and [C, n*C]")
    xc = x if x.is_contiguous() else x.contiguous()
    rows = xc.numel() // C
    out = xc if (inplace and xc is x) else torch.empty_like(xc)
    m = None
    if mask is not None:
        if tuple(mask.shape) != tuple(x.shape[:-1]):
            mask = mask.expand(*x.shape[:-1])
        m = mask.to(torch.float32).contiguous()
    need = lib.of3_transition_rows_workspace_bytes_for(code, rows, C, HID)
    if need < 0 and code == _lib.OF3_DTYPE_BF16 and lib.of3_transition_rows_workspace_bytes_for(_lib.OF3_DTYPE_F32, rows, C, HID) >= 0:
        # widths the bf16 kernels do not serve: the fp32 kernel on widened activations, rounded once at the end
        upd = _swiglu_transition_rows(x.float(), mask, norm_weight, norm_bias, a_weight, b_weight, out_weight, add_residual,
                                      False, _lib.OF3_DTYPE_F32).to(torch.bfloat16)
        if inplace:
            x.copy_(upd)
            return x
        return upd
    if need < 0:
        raise ValueError("single transition: bf16 supports c_in = 384 with a hidden width that is a multiple of 384, "
                         "fp32 c_in <= 512 and hidden <= 2048; got hidden=%d in %s" % (HID, x.dtype))
    ws = _workspace(x.device, max(need, 256))
    keep = [_w(t, x.dtype) for t in (norm_weight, norm_bias, a_weight, b_weight, out_weight)]
    with torch.cuda.device(x.device):
        st = lib.of3_transition_rows_fwd(xc.data_ptr(), None if m is None else m.data_ptr(),
                                         *[k.data_ptr() for k in keep], out.data_ptr(), rows, C, HID,
                                         int(bool(add_residual)), ws.data_ptr(), ws.numel(), code, _stream(x))
    _lib.check(st, "of3_transition_rows_fwd")
    if inplace and out is not x:  # the kernel ran on a contiguous copy of a strided x
        x.copy_(out)
        return x
    return out


def pair_bias(z, norm_weight, norm_bias, weight):
    """Pair bias of AttentionPairBias._prep_bias (attention_pair_bias.py:151-161):
    permute_final_dims(linear_z(layer_norm_z(z)), [2, 0, 1]).  z [*, N, N, C] -> [*, H, N, N] in
    z's dtype; norm_bias may be None (a LayerNorm created without offset); weight is [H, C]."""
    code = _require_gpu(z, "z")
    lib = _lib.load()
    z4, lead = _flatten_pair(z)
    B, N, _, C = z4.shape
    H = weight.shape[0]
    if tuple(weight.shape) != (H, C):
        raise ValueError("pair-bias weight must be [no_heads, c_z]")
    bf16_widths = C in (64, 128) and H <= 32
    fp32_widths = C <= 256 and H <= 64
    if code == _lib.OF3_DTYPE_BF16 and not bf16_widths and fp32_widths:
        # widths the bf16 kernel does not serve: the fp32 kernel on widened activations, rounded once at the end
        return pair_bias(z.float(), norm_weight, norm_bias, weight).to(torch.bfloat16)
    served = bf16_widths if code == _lib.OF3_DTYPE_BF16 else fp32_widths
    nw, w = _w(norm_weight, z.dtype), _w(weight, z.dtype)
    nb = None if norm_bias is None else _w(norm_bias, z.dtype)
    out = torch.empty(B, H, N, N, dtype=z.dtype, device=z.device)
    with torch.cuda.device(z.device):
        st = lib.of3_pair_bias_fwd(z4.data_ptr(), _lib.strides3(z4.stride()[:3]), nw.data_ptr(),
                                   None if nb is None else nb.data_ptr(), w.data_ptr(), out.data_ptr(), B, N, C, H,
                                   code, _stream(z))
    if st == _lib.OF3_EINVAL and not served:
        raise ValueError("pair bias: bf16 supports c_z 64 or 128 and up to 32 heads, fp32 c_z <= 256 and up to 64 "
                         "heads; got c_z=%d heads=%d in %s" % (C, H, z.dtype))
    _lib.check(st, "of3_pair_bias_fwd")
    return out.view(*lead, H, N, N) if len(lead) != 1 else out


def layer_norm(x, weight, bias):
    """LayerNorm over the last dimension (eps 1e-5), the closing step of TemplatePairStack.forward
    (template_module.py:376).  Returns a new contiguous tensor of x's shape and dtype."""
    code = _require_gpu(x, "x")
    lib = _lib.load()
    C = x.shape[-1]
    bf16_widths = C in (64, 128)
    if code == _lib.OF3_DTYPE_BF16 and not bf16_widths and C <= 256:
        return layer_norm(x.float(), weight, bias).to(torch.bfloat16)  # the fp32 kernel, rounded once at the end
    served = bf16_widths if code == _lib.OF3_DTYPE_BF16 else C <= 256
    xc = x.contiguous()
    rows = xc.numel() // C
    out = torch.empty_like(xc)
    w, b = _w(weight, x.dtype), _w(bias, x.dtype)
    with torch.cuda.device(x.device):
        st = lib.of3_layer_norm_fwd(xc.data_ptr(), w.data_ptr(), b.data_ptr(), out.data_ptr(), rows, C, code,
                                    _stream(x))
    if st == _lib.OF3_EINVAL and not served:
        raise ValueError("layer norm: bf16 supports 64 or 128 channels, fp32 up to 256; got %d in %s" % (C, x.dtype))
    _lib.check(st, "of3_layer_norm_fwd")
    return out


def template_tail(t, norm_weight, norm_bias, linear_t_weight, apply_layer_norm: bool = True):
    """Tail of TemplateEmbedderAllAtom.forward (template_module.py:462-465), with the template
    stack's closing LayerNorm (:376) fused in when apply_layer_norm is set:
    linear_t(relu(sum_T LN(t) / T)).  t [*, T, N, N, C_t] -> [*, N, N, C_z] in t's dtype."""
    code = _require_gpu(t, "t")
    lib = _lib.load()
    if t.dim() < 4:
        raise ValueError("t must be [*, N_templ, N, N, C_t]")
    tc = t.contiguous()
    lead = tc.shape[:-4]
    T, N, N2, CT = tc.shape[-4:]
    if N != N2:
        raise ValueError("t must be square in its two token dimensions")
    B = 1
    for d in lead:
        B *= d
    CZ = linear_t_weight.shape[0]
    if tuple(linear_t_weight.shape) != (CZ, CT):
        raise ValueError("linear_t weight must be [c_z, c_t]")
    bf16_widths = CT == 64 and CZ == 128
    fp32_widths = CT <= 256 and CZ <= 4096
    if code == _lib.OF3_DTYPE_BF16 and not bf16_widths and fp32_widths:
        # the fp32 kernel on widened activations, rounded once at the end
        return template_tail(t.float(), norm_weight, norm_bias, linear_t_weight, apply_layer_norm).to(torch.bfloat16)
    served = bf16_widths if code == _lib.OF3_DTYPE_BF16 else fp32_widths
    w = _w(linear_t_weight, t.dtype)
    nw = _w(norm_weight, t.dtype) if apply_layer_norm else None
    nb = _w(norm_bias, t.dtype) if apply_layer_norm else None
    out = torch.empty(*lead, N, N, CZ, dtype=t.dtype, device=t.device)
    with torch.cuda.device(t.device):
        st = lib.of3_template_tail_fwd(tc.data_ptr(), None if nw is None else nw.data_ptr(),
                                       None if nb is None else nb.data_ptr(), w.data_ptr(), out.data_ptr(), B, T,
                                       N * N, CT, CZ, 1 if apply_layer_norm else 0, code, _stream(t))
    if st == _lib.OF3_EINVAL and not served:
        raise ValueError("template tail: bf16 supports c_t = 64 with c_z = 128, fp32 c_t <= 256; got c_t=%d c_z=%d "
                         "in %s" % (CT, CZ, t.dtype))
    _lib.check(st, "of3_template_tail_fwd")
    return out


def attention_pair_bias(a, z, mask, norm_a_weight, norm_a_bias, norm_z_weight, norm_z_bias, z_weight, q_weight,
                        q_bias, k_weight, v_weight, g_weight, o_weight, no_heads: int, inf: float = 1e9,
                        add_residual: bool = False, inplace: bool = False, _bias=None):
    """AttentionPairBias.forward of the trunk (attention_pair_bias.py:189-244): attention over
    the single representation a [*, N, C_s] with the pair bias of z [*, N, N, C_z] and the key
    mask [*, N].  Returns the update (or a + update with add_residual; inplace writes into a).
    bf16: C_s = no_heads * head width = 384; fp32: C_s <= 512."""
    code = _require_gpu(a, "a")
    lib = _lib.load()
    bias = _bias if _bias is not None else pair_bias(z, norm_z_weight, norm_z_bias, z_weight)  # [*, H, N, N]
    if bias.dtype != a.dtype:
        bias = bias.to(a.dtype)
    lead = a.shape[:-2]
    N, CS = a.shape[-2:]
    B = 1
    for d in lead:
        B *= d
    H = no_heads
    HD = q_weight.shape[0]
    if HD % H or tuple(q_weight.shape) != (HD, CS) or tuple(o_weight.shape) != (CS, HD):
        raise ValueError("attention_pair_bias: weights must be [H*c, C_s] and linear_o [C_s, H*c]")
    D = HD // H
    if tuple(bias.shape[-3:]) != (H, N, N) or bias.numel() != B * H * N * N:
        raise ValueError("attention_pair_bias: z must be [*, N, N, C_z] with a's leading dimensions")
    ac = a if a.is_contiguous() else a.contiguous()
    out = ac if (inplace and ac is a) else torch.empty_like(ac)
    m = None
    if mask is not None:
        m = mask.to(torch.float32).expand(*lead, N).contiguous()
    need = lib.of3_attn_pair_bias_workspace_bytes_for(code, B, N, CS, H, D)
    if need < 0 and code == _lib.OF3_DTYPE_BF16 and lib.of3_attn_pair_bias_workspace_bytes_for(_lib.OF3_DTYPE_F32, B, N, CS, H, D) >= 0:
        # widths the bf16 kernels do not serve: the fp32 kernels on widened activations, rounded once at the end
        upd = attention_pair_bias(a.float(), z, mask, norm_a_weight, norm_a_bias, norm_z_weight, norm_z_bias, z_weight,
                                  q_weight, q_bias, k_weight, v_weight, g_weight, o_weight, no_heads, inf=inf,
                                  add_residual=add_residual, inplace=False, _bias=bias.float()).to(torch.bfloat16)
        if inplace:
            a.copy_(upd)
            return a
        return upd
    if need < 0:
        raise ValueError("attention_pair_bias: bf16 supports C_s = no_heads * c = 384 with c a multiple of 8 up to "
                         "24, fp32 C_s <= 512 and c <= 64; got C_s=%d heads=%d c=%d in %s" % (CS, H, D, a.dtype))
    ws = _workspace(a.device, need)
    w = [_w(t, a.dtype) for t in (norm_a_weight, norm_a_bias, q_weight, q_bias, k_weight, v_weight, g_weight, o_weight)]
    with torch.cuda.device(a.device):
        st = lib.of3_attn_pair_bias_fwd(ac.data_ptr(), bias.data_ptr(), None if m is None else m.data_ptr(),
                                        *[t.data_ptr() for t in w], out.data_ptr(), B, N, CS, H, D, float(inf),
                                        1 if add_residual else 0, ws.data_ptr(), ws.numel(), code, _stream(a))
    _lib.check(st, "of3_attn_pair_bias_fwd")
    if inplace and out is not a:  # the kernel ran on a contiguous copy of a strided a
        a.copy_(out)
        return a
    return out

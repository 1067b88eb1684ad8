"""Float64 brute-force statement of the pair-stack math.  TEST INFRASTRUCTURE ONLY.

Written from the index formulas of the path (one Python loop per free index,
numpy float64 dot products over the contracted one), deliberately sharing no
code and no library routine (no layer_norm, no einsum, no softmax) with
oracle/pairstack_oracle.py, so that a dropped term, a swapped index or a
transposed operand in the oracle shows up as a mismatch.  Usable only for
tiny N.

Index formulas and where the reference states them:
  LayerNorm              normalization.py:70-84   y = (x-mean)/sqrt(var_biased+eps)*w+b
  a, b projections       tmu.py:487-493           a = mask * sigmoid(zn Wag^T) * (zn Wap^T)
  outgoing contraction   tmu.py:77-79,95          x[i,j,c] = sum_k a[i,k,c] b[j,k,c]
  incoming contraction   tmu.py:81-82,95          x[i,j,c] = sum_k a[k,i,c] b[k,j,c]
  trimul output          tmu.py:498-501           (LN_out(x) Wz^T) * sigmoid(zn Wg^T)
  attention logits       attention.py:123-127     s = q.k/sqrt(c) + inf*(mask-1) + tb
  triangle bias          tri_att.py:137-140       tb[h,q,k] = (xn[q,k,:] Wz^T)[h]
  gating / output        attention.py:288-302     (o*sigmoid(xn Wg^T)) Wo^T, channel = h*c+d
"""

from __future__ import annotations

import math

import numpy as np


def _f64(t):
    return np.asarray(t.detach().cpu().double().numpy() if hasattr(t, "detach") else t, dtype=np.float64)


def _ln(v, w, b, eps=1e-5):
    mu = v.sum() / v.size
    var = ((v - mu) ** 2).sum() / v.size
    return (v - mu) / math.sqrt(var + eps) * w + b


def _sig(v):
    return 1.0 / (1.0 + np.exp(-v))


def trimul_update(z, mask, p, outgoing):
    """z: [N, N, C], mask: [N, N] -> [N, N, C] float64."""
    z = _f64(z)
    mask = _f64(mask)
    P = {k: _f64(v) for k, v in p.items()}
    N, _, C = z.shape
    Ch = P["linear_a_p.weight"].shape[0]
    zn = np.zeros_like(z)
    a = np.zeros((N, N, Ch))
    b = np.zeros((N, N, Ch))
    for i in range(N):
        for j in range(N):
            zn[i, j] = _ln(z[i, j], P["layer_norm_in.weight"], P["layer_norm_in.bias"])
            a[i, j] = mask[i, j] * _sig(P["linear_a_g.weight"] @ zn[i, j]) * (P["linear_a_p.weight"] @ zn[i, j])
            b[i, j] = mask[i, j] * _sig(P["linear_b_g.weight"] @ zn[i, j]) * (P["linear_b_p.weight"] @ zn[i, j])
    out = np.zeros((N, N, C))
    for i in range(N):
        for j in range(N):
            x = np.zeros(Ch)
            for k in range(N):
                if outgoing:
                    x += a[i, k] * b[j, k]
                else:
                    x += a[k, i] * b[k, j]
            xn = _ln(x, P["layer_norm_out.weight"], P["layer_norm_out.bias"])
            out[i, j] = (P["linear_z.weight"] @ xn) * _sig(P["linear_g.weight"] @ zn[i, j])
    return out


def triattn_update(x, mask, p, no_heads, starting=True, inf=1e9):
    """x: [I, J, C] (I == J), mask: [I, J] -> [I, J, C] float64.

    The ending node is stated directly on the un-transposed tensor:
    out[i,j] attends over k with q from x[i,j], k/v from x[k,j], key mask
    mask[k,j] and triangle bias from x[k,i]  (tri_att.py:126-128,164-165).
    """
    x = _f64(x)
    mask = _f64(mask)
    P = {k: _f64(v) for k, v in p.items()}
    N, _, C = x.shape
    H = no_heads
    Wq, Wk, Wv, Wg = (P["mha.linear_%s.weight" % n] for n in "qkvg")
    Wo, Wb = P["mha.linear_o.weight"], P["linear_z.weight"]
    c = Wq.shape[0] // H
    xn = np.zeros_like(x)
    for i in range(N):
        for j in range(N):
            xn[i, j] = _ln(x[i, j], P["layer_norm.weight"], P["layer_norm.bias"])
    out = np.zeros((N, N, C))
    for i in range(N):
        for j in range(N):
            qv = (Wq @ xn[i, j]) / math.sqrt(c)
            gv = _sig(Wg @ xn[i, j])
            o = np.zeros(H * c)
            for h in range(H):
                s = np.zeros(N)
                vals = np.zeros((N, c))
                for k in range(N):
                    if starting:
                        src, mk, bsrc = xn[i, k], mask[i, k], xn[j, k]
                    else:
                        src, mk, bsrc = xn[k, j], mask[k, j], xn[k, i]
                    kv = (Wk @ src)[h * c:(h + 1) * c]
                    vals[k] = (Wv @ src)[h * c:(h + 1) * c]
                    qk = qv[h * c:(h + 1) * c] @ kv
                    tb = (Wb @ bsrc)[h]
                    if mk == 1.0:
                        s[k] = qk + tb
                    else:
                        # The reference adds the mask bias to the logit first, then the
                        # triangle bias (attention.py:126-127), in float32: -1e9 absorbs
                        # any |logit| < 32 (ulp(1e9) = 64), which is what makes a fully
                        # masked row a uniform average.  float64 would not absorb, so
                        # these two adds are rounded to float32 here.
                        t = np.float32(np.float32(qk) + np.float32(inf * (mk - 1.0)))
                        s[k] = float(np.float32(t + np.float32(tb)))
                s = s - s.max()
                w = np.exp(s)
                w = w / w.sum()
                o[h * c:(h + 1) * c] = w @ vals
            out[i, j] = Wo @ (o * gv)
    return out


def transition_update(x, mask, p):
    """(silu(LN(x) Wa^T) * (LN(x) Wb^T)) Wout^T * mask, one position at a time
    (transition.py:261-271, activations.py:60-61); silu(t) = t / (1 + exp(-t))."""
    x = _f64(x)
    shape = x.shape
    c = shape[-1]
    xf = x.reshape(-1, c)
    mf = np.ones(xf.shape[0]) if mask is None else _f64(mask).reshape(-1)
    lw, lb = _f64(p["layer_norm.weight"]), _f64(p["layer_norm.bias"])
    wa, wb, wo = _f64(p["swiglu.linear_a.weight"]), _f64(p["swiglu.linear_b.weight"]), _f64(p["linear_out.weight"])
    out = np.zeros_like(xf)
    for r in range(xf.shape[0]):
        xn = _ln(xf[r], lw, lb)
        h = np.zeros(wa.shape[0])
        for j in range(wa.shape[0]):
            ta = float(np.dot(wa[j], xn))
            tb = float(np.dot(wb[j], xn))
            h[j] = ta / (1.0 + math.exp(-ta)) * tb
        for co in range(c):
            out[r, co] = float(np.dot(wo[co], h)) * mf[r]
    return out.reshape(shape)


def pair_bias(z, p):
    """float64 loops: out[h, i, j] = sum_c LN(z[i, j, :])[c] * W[h, c] for z [N, N, C]."""
    z = np.asarray(z, dtype=np.float64)
    w = np.asarray(p["linear_z.weight"], dtype=np.float64)
    g = np.asarray(p["layer_norm_z.weight"], dtype=np.float64)
    b = np.asarray(p["layer_norm_z.bias"], dtype=np.float64) if "layer_norm_z.bias" in p else np.zeros_like(g)
    n, _, c = z.shape
    out = np.zeros((w.shape[0], n, n))
    for i in range(n):
        for j in range(n):
            x = z[i, j]
            mu = x.sum() / c
            var = ((x - mu) ** 2).sum() / c
            xn = (x - mu) / np.sqrt(var + 1e-5) * g + b
            for h in range(w.shape[0]):
                out[h, i, j] = (xn * w[h]).sum()
    return out


def template_tail(t, ln_w, ln_b, w):
    """float64 loops: out[i, j, :] = W @ relu(mean_T LN(t[T, i, j, :])) for t [T, N, N, C]
    (template_module.py:376 and :462-465)."""
    t = np.asarray(t, dtype=np.float64)
    g = np.asarray(ln_w, dtype=np.float64)
    b = np.asarray(ln_b, dtype=np.float64)
    w = np.asarray(w, dtype=np.float64)
    nt, n, _, c = t.shape
    out = np.zeros((n, n, w.shape[0]))
    for i in range(n):
        for j in range(n):
            acc = np.zeros(c)
            for k in range(nt):
                acc += _ln(t[k, i, j], g, b)
            acc = np.maximum(acc / nt, 0.0)
            for o in range(w.shape[0]):
                out[i, j, o] = (w[o] * acc).sum()
    return out


def attention_pair_bias(a, z, mask, p, no_heads, inf=1e9):
    """float64 loops over (head, query, key) for a [N, C_s], z [N, N, C_z], mask [N]
    (attention_pair_bias.py:189-244, attention.py:94-135, :265-302)."""
    a = np.asarray(a, dtype=np.float64)
    z = np.asarray(z, dtype=np.float64)
    P = {k: np.asarray(v, dtype=np.float64) for k, v in p.items()}
    n, cs = a.shape
    hc = P["mha.linear_q.weight"].shape[0]
    c = hc // no_heads
    mask = np.ones(n) if mask is None else np.asarray(mask, dtype=np.float64)
    an = np.stack([_ln(a[i], P["layer_norm_a.weight"], P["layer_norm_a.bias"]) for i in range(n)])
    zb_b = P.get("layer_norm_z.bias", np.zeros_like(P["layer_norm_z.weight"]))
    q = np.zeros((n, hc)); k = np.zeros((n, hc)); v = np.zeros((n, hc)); g = np.zeros((n, hc))
    for i in range(n):
        for o in range(hc):
            q[i, o] = ((an[i] * P["mha.linear_q.weight"][o]).sum() + P["mha.linear_q.bias"][o]) / math.sqrt(c)
            k[i, o] = (an[i] * P["mha.linear_k.weight"][o]).sum()
            v[i, o] = (an[i] * P["mha.linear_v.weight"][o]).sum()
            g[i, o] = _sig((an[i] * P["mha.linear_g.weight"][o]).sum())
    og = np.zeros((n, hc))
    for h in range(no_heads):
        sl = slice(h * c, (h + 1) * c)
        for i in range(n):
            logits = np.zeros(n)
            for j in range(n):
                zn = _ln(z[i, j], P["layer_norm_z.weight"], zb_b)
                logits[j] = (q[i, sl] * k[j, sl]).sum() + inf * (mask[j] - 1) + (zn * P["linear_z.weight"][h]).sum()
            w = np.exp(logits - logits.max())
            w /= w.sum()
            for d in range(c):
                og[i, h * c + d] = (w * v[:, h * c + d]).sum() * g[i, h * c + d]
    out = np.zeros((n, cs))
    for i in range(n):
        for o in range(cs):
            out[i, o] = (og[i] * P["mha.linear_o.weight"][o]).sum()
    return out

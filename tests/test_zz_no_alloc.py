"""of3_trimul_fwd_static, the entry point that allocates nothing (its scratch is an array built into
the library): called through the C ABI it must give what of3_trimul_fwd gives with a caller's
workspace, bit for bit (same kernels, same order of operations), also on a second call with a
smaller input that finds the first call's contents in the scratch, and the result must match the
CPU oracle to the bf16 bound of the other parity tests (max|err| <= 2e-2 * max|want|).  Problems
beyond the built-in scratch are refused before anything is launched."""
import pytest
import torch

from gpu_util import _lib, lib, report, s3, stream
from oracle import pairstack_oracle as orc

DEV = "cuda"
NAMES = ("layer_norm_in.weight", "layer_norm_in.bias", "layer_norm_out.weight", "layer_norm_out.bias",
         "linear_a_p.weight", "linear_a_g.weight", "linear_b_p.weight", "linear_b_g.weight", "linear_g.weight",
         "linear_z.weight")


def _case(seed, B, N, C, dtype, outgoing):
    gen = torch.Generator().manual_seed(seed)
    p = orc.make_trimul_params(gen, C, C)
    z = orc.make_pair_input(seed + 1, (B,), N, C)
    mask = (torch.rand(B, N, N, generator=gen) > 0.2).float()
    if dtype == torch.bfloat16:
        p = {k: orc.round_bf16(v) for k, v in p.items()}
        z = orc.round_bf16(z)
    want = z + orc.trimul_update(z, mask, p, outgoing)
    dp = [p[k].to(DEV).to(dtype).contiguous() for k in NAMES]
    return z.to(DEV).to(dtype), mask.to(DEV), dp, want


def _both(L, B, N, C, dtype, outgoing, seed):
    code = _lib.OF3_DTYPE_BF16 if dtype == torch.bfloat16 else _lib.OF3_DTYPE_F32
    z, mask, dp, want = _case(seed, B, N, C, dtype, outgoing)
    w = [t.data_ptr() for t in dp]
    need = L.of3_trimul_workspace_bytes_for(code, B, N, C, C)
    assert 0 < need <= _lib.OF3_STATIC_SCRATCH_BYTES
    ws = torch.empty(need, dtype=torch.uint8, device=DEV)
    ref = torch.empty_like(z)
    got = torch.empty_like(z)
    print("trimul static vs workspace: B=%d N=%d C=%d %s outgoing=%d" % (B, N, C, dtype, outgoing), flush=True)
    st = L.of3_trimul_fwd(z.data_ptr(), s3(z), mask.data_ptr(), s3(mask), *w, ref.data_ptr(), B, N, C, C, outgoing, 1,
                          ws.data_ptr(), ws.numel(), code, stream())
    _lib.check(st, "of3_trimul_fwd")
    st = L.of3_trimul_fwd_static(z.data_ptr(), s3(z), mask.data_ptr(), s3(mask), *w, got.data_ptr(), B, N, C, C,
                                 outgoing, 1, code, stream())
    _lib.check(st, "of3_trimul_fwd_static")
    torch.cuda.synchronize()
    assert torch.equal(got, ref), "static-scratch result differs from the workspace entry point's"
    if dtype == torch.bfloat16:
        report("trimul static vs oracle", got.cpu(), want, atol=2e-2 * float(want.abs().max()))
    else:
        report("trimul static vs oracle (fp32)", got.cpu(), want, atol=1e-4)


@pytest.mark.gpu
def test_static_scratch_matches_workspace_entry_point_twice():
    L = lib()
    # the largest bf16 problem the scratch takes (48 MiB), then a smaller and ragged one that finds
    # the first call's a, b and x in the scratch; then the template shape and the fp32 kernels
    _both(L, 1, 256, 128, torch.bfloat16, 1, seed=11)
    _both(L, 1, 100, 128, torch.bfloat16, 0, seed=12)
    _both(L, 2, 72, 64, torch.bfloat16, 1, seed=13)
    _both(L, 1, 96, 128, torch.float32, 1, seed=14)
    _both(L, 1, 40, 128, torch.float32, 0, seed=15)


@pytest.mark.gpu
def test_static_entry_point_under_graph_capture_after_an_eager_call():
    """The callers the entry point is for include code under stream capture.  The first call on a device
    does look-ups that a capture does not allow, so one eager call comes first; after it the entry point
    issues kernel launches only and can be captured.  Every replay (with eager work and synchronisations
    in between) must reproduce the eager result bit for bit."""
    L = lib()
    B, N, C = 1, 96, 128
    code = _lib.OF3_DTYPE_BF16
    z, mask, dp, _ = _case(21, B, N, C, torch.bfloat16, 1)
    w = [t.data_ptr() for t in dp]
    eager = torch.empty_like(z)
    print("trimul static under capture: B=%d N=%d C=%d" % (B, N, C), flush=True)
    st = L.of3_trimul_fwd_static(z.data_ptr(), s3(z), mask.data_ptr(), s3(mask), *w, eager.data_ptr(), B, N, C, C, 1, 1,
                                 code, stream())
    _lib.check(st, "of3_trimul_fwd_static (eager warm-up)")
    torch.cuda.synchronize()
    z_static = z.clone()
    out_static = torch.empty_like(z)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        st = L.of3_trimul_fwd_static(z_static.data_ptr(), s3(z_static), mask.data_ptr(), s3(mask), *w,
                                     out_static.data_ptr(), B, N, C, C, 1, 1, code, stream())
    _lib.check(st, "of3_trimul_fwd_static (captured)")
    for rep in range(3):
        # eager work between the replays that also uses the built-in scratch (a smaller problem)
        z2, m2, dp2, _ = _case(22 + rep, 1, 40, C, torch.bfloat16, 0)
        o2 = torch.empty_like(z2)
        st = L.of3_trimul_fwd_static(z2.data_ptr(), s3(z2), m2.data_ptr(), s3(m2), *[t.data_ptr() for t in dp2],
                                     o2.data_ptr(), 1, 40, C, C, 0, 1, code, stream())
        _lib.check(st, "of3_trimul_fwd_static (eager between replays)")
        torch.cuda.synchronize()
        out_static.zero_()
        z_static.copy_(z)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out_static, eager), "replay %d differs from the eager call" % rep


def test_static_scratch_rejects_what_does_not_fit():
    """No GPU needed: sizes are checked before the first HIP call."""
    L = lib()
    fake = 0x10000
    zs = _lib.strides3((384 * 384 * 128, 384 * 128, 128))

    def call(N, C=128, dtype=_lib.OF3_DTYPE_BF16):
        return L.of3_trimul_fwd_static(fake, zs, None, None, *([fake] * 10), fake, 1, N, C, C, 1, 1, dtype, None)

    assert L.of3_trimul_workspace_bytes(1, 256, 128, 128) == _lib.OF3_STATIC_SCRATCH_BYTES
    assert call(257) == _lib.OF3_ESTATIC
    assert call(384) == _lib.OF3_ESTATIC
    assert call(200, dtype=_lib.OF3_DTYPE_F32) == _lib.OF3_ESTATIC
    # fp32 at C = CH = 128: the rule is the workspace size, not B*CH*N*N (N = 143..160 are below 2^22 there)
    f32 = _lib.OF3_DTYPE_F32
    assert L.of3_trimul_workspace_bytes_for(f32, 1, 142, 128, 128) <= _lib.OF3_STATIC_SCRATCH_BYTES
    assert L.of3_trimul_workspace_bytes_for(f32, 1, 143, 128, 128) > _lib.OF3_STATIC_SCRATCH_BYTES
    assert call(143, dtype=f32) == _lib.OF3_ESTATIC
    assert call(160, dtype=f32) == _lib.OF3_ESTATIC
    assert call(64, C=96) == _lib.OF3_EINVAL
    assert call(64, dtype=5) == _lib.OF3_EINVAL
    assert b"OF3_STATIC_SCRATCH_BYTES" in L.of3_status_string(_lib.OF3_ESTATIC)

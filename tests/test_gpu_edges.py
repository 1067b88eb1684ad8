"""Edge cases of the HIP path: smallest and ragged sizes, strided and sliced inputs, mask dtypes,
other streams, run-to-run determinism.  Same oracle and tolerances as tests/test_gpu_parity.py."""
import pytest
import torch

from gpu_util import lib  # noqa: F401
from oracle import pairstack_oracle as orc
from test_gpu_parity import _check, _load, _round_params, DEV

import of3pair

pytestmark = pytest.mark.gpu


def _block(c, d, seed=0):
    p = _round_params(orc.make_block_params(seed, c, c, d, 4))
    return _load(of3pair.PairStack(c, c, d, 4), p), p


@pytest.mark.parametrize("n", [1, 2, 31, 33, 129, 200])
def test_block_small_and_ragged_sizes(n):
    """N = 1 (a single token), N below, at and just above the 32-key and 128-position tile sizes."""
    lib()
    m, p = _block(128, 32, seed=30 + n)
    gen = torch.Generator().manual_seed(n)
    z = orc.round_bf16(torch.randn(2, n, n, 128, generator=gen))
    mask = (torch.rand(2, n, n, generator=gen) > 0.15).float()
    mask[0] = 1.0
    print("ragged block n =", n, flush=True)
    got = m(z.to(DEV).to(torch.bfloat16), mask.to(DEV))
    want = orc.pair_stack_block(z, mask, p, 4)
    _check("block n=%d" % n, got, want, rms_rel=1.2e-2)


@pytest.mark.parametrize("seed", range(8))
def test_block_random_ragged_shapes(seed):
    """Seeded random token counts (every width of the ragged row ends: 8, 16, 32, 64 and 128 columns),
    batch sizes, both channel widths, random and tail-padding masks; out of place and in place."""
    lib()
    gen = torch.Generator().manual_seed(9000 + seed)
    wide = seed % 2 == 0
    c, d = (128, 32) if wide else (64, 16)
    n = int(torch.randint(3, 190, (1,), generator=gen)) if seed < 6 else (int(torch.randint(129, 140, (1,), generator=gen)) if seed == 6 else 161)
    b = int(torch.randint(1, 4, (1,), generator=gen))
    m, p = _block(c, d, seed=9100 + seed)
    z = orc.round_bf16(torch.randn(b, n, n, c, generator=gen))
    if seed % 3 == 0:
        mask = orc.tail_padding_mask((b,), n, torch.randint(0, max(1, n // 4), (b,), generator=gen))
    else:
        mask = (torch.rand(b, n, n, generator=gen) > 0.2).float()
    print("random ragged block: seed", seed, "c", c, "n", n, "batch", b, flush=True)
    zg = z.to(DEV).to(torch.bfloat16)
    want = orc.pair_stack_block(z, mask, p, 4)
    got = m(zg, mask.to(DEV))
    _check("random block seed %d n=%d" % (seed, n), got, want, rms_rel=1.2e-2)
    res = m(zg, mask.to(DEV), inplace_safe=True)
    assert res.data_ptr() == zg.data_ptr() and torch.equal(res, got), "in place and out of place differ"


def test_fully_masked_input():
    """mask == 0 everywhere: trimul contributes (LN_out.bias Wz^T)*gate, attention averages v uniformly."""
    lib()
    n = 48
    m, p = _block(64, 16, seed=41)
    z = orc.round_bf16(orc.make_pair_input(42, (1,), n, 64))
    mask = torch.zeros(1, n, n)
    got = m(z.to(DEV).to(torch.bfloat16), mask.to(DEV))
    _check("all masked", got, orc.pair_stack_block(z, mask, p, 4), rms_rel=1.2e-2)


def test_strided_batch_and_sliced_inputs():
    """A batch taken as every other element of a larger tensor and a square window of a larger pair
    tensor: the kernels follow the strides, nothing is copied for the batch case."""
    lib()
    n = 40
    gen = torch.Generator().manual_seed(50)
    p = _round_params(orc.make_trimul_params(gen, 128, 128))
    m = _load(of3pair.TriangleMultiplicationIncoming(128, 128), p)
    big = orc.round_bf16(torch.randn(4, n, n, 128, generator=gen))
    bg = big.to(DEV).to(torch.bfloat16)
    got = m(bg[::2])                                    # batch stride 2*N*N*C
    _check("strided batch", got, orc.trimul_update(big[::2], None, p, False))
    win = bg[1, 4:36, 4:36, :]                          # row stride N*C, 32 x 32 window
    got = m(win)
    _check("window", got, orc.trimul_update(big[1, 4:36, 4:36, :], None, p, False))
    pa = _round_params(orc.make_triattn_params(gen, 128, 32, 4))
    a = _load(of3pair.TriangleAttention(128, 32, 4, starting=False), pa)
    got = a(win, mask=torch.ones(32, 32, device=DEV))
    _check("window attention", got, orc.triattn_update(big[1, 4:36, 4:36, :], None, pa, 4, starting=False), rms_rel=6e-3)


@pytest.mark.parametrize("dtype", [torch.bool, torch.int32, torch.bfloat16, torch.float64])
def test_mask_dtypes(dtype):
    """The reference accepts 0/1 masks of any dtype (tmu.py:485, tri_att.py:134)."""
    lib()
    n = 36
    m, p = _block(128, 32, seed=60)
    gen = torch.Generator().manual_seed(61)
    z = orc.round_bf16(torch.randn(1, n, n, 128, generator=gen))
    mask = (torch.rand(1, n, n, generator=gen) > 0.3)
    got = m(z.to(DEV).to(torch.bfloat16), mask.to(dtype).to(DEV))
    _check("mask " + str(dtype), got, orc.pair_stack_block(z, mask.float(), p, 4), rms_rel=1.2e-2)


def test_runs_on_the_current_stream_and_is_deterministic():
    lib()
    n = 96
    m, p = _block(128, 32, seed=70)
    z = orc.round_bf16(orc.make_pair_input(71, (1,), n, 128)).to(DEV).to(torch.bfloat16)
    mask = orc.tail_padding_mask((1,), n, 7).to(DEV)
    ref = m(z, mask)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        outs = [m(z, mask) for _ in range(3)]
    side.synchronize()
    for o in outs:
        assert torch.equal(o, ref), "results differ between runs / streams"


def test_pair_block_in_a_hip_graph_replays_like_eager():
    """The library allocates nothing and synchronises nothing, so a whole PairBlock (pair stack +
    transition) can be captured into a HIP graph once its one-time set-up has run.  The graph is
    replayed several times with eager work and synchronisations in between; every replay must
    reproduce the eager result bit for bit."""
    lib()
    c, n = 128, 96
    gen = torch.Generator().manual_seed(77)
    p = _round_params(orc.make_block_params(3, c, c, 32, 4))
    p.update({"pair_transition." + k: orc.round_bf16(v) for k, v in orc.make_transition_params(gen, c, 4).items()})
    blk = of3pair.PairBlock(c, c, 32, 4, "swiglu", 4, 0.0, False, 1e9)
    blk.load_state_dict(p, strict=True)
    blk = blk.to(DEV).to(torch.bfloat16).eval()
    z0 = orc.round_bf16(orc.make_pair_input(23, (1,), n, c)).to(DEV).to(torch.bfloat16)
    mask = orc.tail_padding_mask((1,), n, 7).to(DEV)
    eager = blk(z0, mask)                       # also the warm-up: workspace and launch geometry exist now
    torch.cuda.synchronize()
    z_static = z0.clone()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out_static = blk(z_static, mask)
    for rep in range(3):
        z_static.copy_(z0)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out_static, eager), "replay %d differs from the eager result" % rep
        # eager work between the replays, on the same buffers the library uses
        other = blk(z0 * 0.5, mask)
        assert torch.isfinite(other).all()
        torch.cuda.synchronize()
    # new input through the same graph
    z1 = orc.round_bf16(orc.make_pair_input(24, (1,), n, c)).to(DEV).to(torch.bfloat16)
    z_static.copy_(z1)
    graph.replay()
    torch.cuda.synchronize()
    assert torch.equal(out_static, blk(z1, mask))


def test_outgrown_workspace_stays_valid_for_a_captured_graph():
    """A graph captured at a small N keeps pointing into the scratch buffer of its capture (the capture
    stream has a buffer of its own); later eager calls at a larger N need more scratch on their stream.
    The eager buffer they outgrow was never handed to a capture and is freed, not hoarded; the graph's
    buffer is untouched, so the replay still reproduces the eager result of the small problem."""
    from of3pair import functional as F3

    lib()
    torch.cuda.synchronize()
    F3.release_workspaces()  # earlier tests have grown the scratch already; no graph of theirs is replayed again
    blk, _ = _block(128, 32, seed=5)
    z_small = orc.round_bf16(orc.make_pair_input(31, (1,), 40, 128)).to(DEV).to(torch.bfloat16)
    m_small = torch.ones(1, 40, 40, device=DEV)
    eager_small = blk(z_small, m_small)
    torch.cuda.synchronize()
    z_static = z_small.clone()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out_static = blk(z_static, m_small)
    for n in (96, 160, 224):  # eager calls of rising length: each outgrows the eager stream's scratch
        z_big = orc.round_bf16(orc.make_pair_input(32, (1,), n, 128)).to(DEV).to(torch.bfloat16)
        big = blk(z_big, torch.ones(1, n, n, device=DEV))
        assert torch.isfinite(big).all()
        assert len(F3._retired) == 0, "an eager buffer no capture has used is freed when it is outgrown"
    filler = torch.full((64 << 20,), 7, dtype=torch.uint8, device=DEV)  # would land in freed scratch memory
    for rep in range(2):
        z_static.copy_(z_small)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out_static, eager_small), "replay %d after the workspace grew" % rep
    assert int(filler[0]) == 7


def test_workspace_used_by_a_capture_is_kept_when_outgrown():
    """Warm-up and capture on one side stream share that stream's scratch buffer, so the graph points
    into it.  A larger eager call on the same stream outgrows it: the buffer must be kept alive (retired,
    not freed) until release_workspaces(), and the replay must still give the small problem's result."""
    from of3pair import functional as F3

    lib()
    torch.cuda.synchronize()
    F3.release_workspaces()
    blk, _ = _block(128, 32, seed=6)
    z_small = orc.round_bf16(orc.make_pair_input(33, (1,), 40, 128)).to(DEV).to(torch.bfloat16)
    m_small = torch.ones(1, 40, 40, device=DEV)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        eager_small = blk(z_small, m_small)  # allocates the side stream's scratch, eagerly
    side.synchronize()
    z_static = z_small.clone()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        out_static = blk(z_static, m_small)  # same stream, same buffer: now referenced by the graph
    assert len(F3._retired) == 0
    with torch.cuda.stream(side):
        z_big = orc.round_bf16(orc.make_pair_input(34, (1,), 160, 128)).to(DEV).to(torch.bfloat16)
        big = blk(z_big, torch.ones(1, 160, 160, device=DEV))
    side.synchronize()
    assert torch.isfinite(big).all()
    assert len(F3._retired) == 1, "a buffer a captured graph points into is kept until release_workspaces()"
    filler = torch.full((64 << 20,), 7, dtype=torch.uint8, device=DEV)
    for rep in range(2):
        z_static.copy_(z_small)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out_static, eager_small), "replay %d after the workspace grew" % rep
    assert int(filler[0]) == 7
    del graph
    F3.release_workspaces()


def test_bf16_widths_outside_the_mfma_kernels_run_on_the_fp32_kernels():
    """The bf16 MFMA kernels serve the AF3 widths; a bf16 pair tensor of any other width (here
    c_z = 96, c_hidden_mul = 40, 3 heads of 16, transition n = 2) is widened on the device, runs on
    the fp32 kernels and is rounded to bf16 at the end: same interface, in-place contract included."""
    lib()
    c, ch, d, heads, n = 96, 40, 16, 3, 37
    p = _round_params(orc.make_block_params(61, c, ch, d, heads))
    gen = torch.Generator().manual_seed(62)
    p.update({"pair_transition." + k: orc.round_bf16(v) for k, v in orc.make_transition_params(gen, c, 2).items()})
    blk = _load(of3pair.PairBlock(c, ch, d, heads, "swiglu", 2, 0.0, False, 1e9), p)
    z = orc.round_bf16(orc.make_pair_input(63, (2,), n, c))
    mask = orc.tail_padding_mask((2,), n, torch.tensor([5, 0]))
    zg = z.to(DEV).to(torch.bfloat16)
    got = blk(zg, mask.to(DEV))
    assert got.dtype == torch.bfloat16 and torch.equal(zg.float().cpu(), z)
    want = orc.pair_block(z, mask, p, heads)
    _check("odd-width bf16 block", got, want, rms_rel=1.2e-2)
    res = blk(zg, mask.to(DEV), inplace_safe=True)
    assert res.data_ptr() == zg.data_ptr()
    assert torch.equal(res, got)

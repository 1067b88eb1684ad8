"""Host-side mirror of the reference's layer interface, checked without a GPU: constructor
arguments, parameter names and shapes (state-dict compatibility), initialisers, forward
signatures, and that the product path refuses to run without the HIP kernels' device."""
import inspect

import pytest
import torch

import of3pair
from of3pair import layers


def test_trimul_state_dict_names_and_shapes():
    m = of3pair.TriangleMultiplicationOutgoing(128, 128)
    sd = m.state_dict()
    want = {
        "layer_norm_in.weight": (128,), "layer_norm_in.bias": (128,),
        "layer_norm_out.weight": (128,), "layer_norm_out.bias": (128,),
        "linear_a_p.weight": (128, 128), "linear_a_g.weight": (128, 128),
        "linear_b_p.weight": (128, 128), "linear_b_g.weight": (128, 128),
        "linear_g.weight": (128, 128), "linear_z.weight": (128, 128),
    }
    assert {k: tuple(v.shape) for k, v in sd.items()} == want
    assert m._outgoing is True
    assert of3pair.TriangleMultiplicationIncoming(64, 64)._outgoing is False


def test_triattn_state_dict_names_and_shapes():
    m = of3pair.TriangleAttention(128, 32, 4)
    want = {
        "layer_norm.weight": (128,), "layer_norm.bias": (128,), "linear_z.weight": (4, 128),
        "mha.linear_q.weight": (128, 128), "mha.linear_k.weight": (128, 128), "mha.linear_v.weight": (128, 128),
        "mha.linear_o.weight": (128, 128), "mha.linear_g.weight": (128, 128),
    }
    assert {k: tuple(v.shape) for k, v in m.state_dict().items()} == want
    assert m.starting is True and of3pair.TriangleAttentionEndingNode(128, 32, 4).starting is False
    assert m.inf == 1e9


def test_default_initialisers_follow_the_af3_tables():
    torch.manual_seed(0)
    m = of3pair.TriangleMultiplicationOutgoing(128, 128)
    for zero in ("linear_a_g", "linear_b_g", "linear_g", "linear_z"):      # "final" = zeros
        assert getattr(m, zero).weight.abs().max() == 0
    for dflt in ("linear_a_p", "linear_b_p"):                               # LeCun truncated normal
        w = getattr(m, dflt).weight
        assert 0.7 / 128 ** 0.5 < w.std() < 1.3 / 128 ** 0.5
        assert w.abs().max() <= 2.0 / 0.87962566103423978 / 128 ** 0.5 + 1e-6
    a = of3pair.TriangleAttention(128, 32, 4)
    assert a.mha.linear_o.weight.abs().max() == 0 and a.mha.linear_g.weight.abs().max() == 0
    assert a.mha.linear_q.weight.std() > 0 and a.linear_z.weight.std() > 0
    assert m.layer_norm_in.eps == 1e-5 and a.layer_norm.eps == 1e-5


def test_reference_style_init_params_are_accepted():
    spec = {k: {"bias": False, "init": "default"} for k in layers.TRI_MUL_INIT}
    m = of3pair.TriangleMultiplicationOutgoing(64, 64, linear_init_params=spec)
    assert m.linear_z.weight.abs().max() > 0
    with pytest.raises(ValueError):
        of3pair.TriangleMultiplicationOutgoing(64, 64, linear_init_params={**spec, "linear_g": {"bias": True, "init": "final"}})


def test_forward_signatures_match_the_reference():
    tm = inspect.signature(of3pair.TriangleMultiplicativeUpdate.forward)
    assert list(tm.parameters)[1:] == ["z", "mask", "inplace_safe", "use_cueq_triangle_kernels",
                                       "_add_with_inplace", "_inplace_chunk_size"]
    ta = list(inspect.signature(of3pair.TriangleAttention.forward).parameters)[1:]
    assert ta[:7] == ["x", "mask", "chunk_size", "use_deepspeed_evo_attention", "use_cueq_triangle_kernels",
                      "use_lma", "inplace_safe"]
    ctor = list(inspect.signature(of3pair.TriangleAttention.__init__).parameters)[1:]
    assert ctor == ["c_in", "c_hidden", "no_heads", "starting", "inf", "linear_init_params"]


def test_pair_stack_submodule_names():
    ps = of3pair.PairStack(128, 128, 32, 4)
    names = {k.split(".")[0] for k in ps.state_dict()}
    assert names == {"tri_mul_out", "tri_mul_in", "tri_att_start", "tri_att_end"}
    assert ps.tri_att_end.starting is True  # like the reference: a starting module fed the transposed tensor


def test_no_cpu_fallback():
    """The shipped path has no CPU implementation: CPU tensors are refused loudly."""
    m = of3pair.TriangleMultiplicationOutgoing(128, 128).to(torch.bfloat16)
    z = torch.zeros(1, 8, 8, 128, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="GPU"):
        m(z)
    a = of3pair.TriangleAttention(128, 32, 4).to(torch.bfloat16)
    with pytest.raises(RuntimeError, match="GPU"):
        a(z)
    with pytest.raises(RuntimeError, match="GPU"):  # fp32 has no CPU path either
        of3pair.TriangleMultiplicationOutgoing(128, 128)(z.float())


def test_package_does_not_import_the_oracle():
    import sys

    import of3pair.functional  # noqa: F401
    import of3pair.pair_stack  # noqa: F401

    src_dir = of3pair.__path__[0]
    import os
    for fn in os.listdir(src_dir):
        if fn.endswith(".py"):
            text = open(os.path.join(src_dir, fn)).read()
            assert "oracle" not in text, "%s mentions the oracle" % fn

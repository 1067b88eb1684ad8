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
    m = of3pair.TriangleMultiplicationOutgoing(128, 128).to(torch.bfloat16).eval()
    z = torch.zeros(1, 8, 8, 128, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="GPU"):
        m(z)
    a = of3pair.TriangleAttention(128, 32, 4).to(torch.bfloat16).eval()
    with pytest.raises(RuntimeError, match="GPU"):
        a(z)
    with pytest.raises(RuntimeError, match="GPU"):  # fp32 has no CPU path either
        of3pair.TriangleMultiplicationOutgoing(128, 128).eval()(z.float())


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


TEMPLATE_STACK_CFG = dict(c_t=64, c_hidden_tri_att=16, c_hidden_tri_mul=64, no_blocks=2, no_heads=4,
                          transition_type="swiglu", pair_transition_n=2, dropout_rate=0.25, tri_mul_first=True,
                          fuse_projection_weights=False, blocks_per_ckpt=None, inf=1e9, use_reentrant=False,
                          tune_chunk_size=False)


def test_template_modules_take_the_reference_config_and_names():
    """template_pair_stack of the reference's model config (model_config.py:212-230) constructs
    the stack; parameter names are the reference's (blocks.<i>.<PairBlock names>, layer_norm)."""
    stack = of3pair.TemplatePairStack(**TEMPLATE_STACK_CFG)
    names = set(stack.state_dict())
    assert len(stack.blocks) == 2 and stack.blocks[0].tri_mul_first is True
    for i in (0, 1):
        for k in ("tri_mul_out.linear_a_p.weight", "tri_mul_in.layer_norm_out.bias", "tri_att_start.mha.linear_q.weight",
                  "tri_att_end.linear_z.weight", "pair_transition.layer_norm.weight",
                  "pair_transition.swiglu.linear_a.weight", "pair_transition.linear_out.weight"):
            assert "blocks.%d.%s" % (i, k) in names
    assert {"layer_norm.weight", "layer_norm.bias"} <= names
    assert tuple(stack.state_dict()["blocks.1.pair_transition.swiglu.linear_b.weight"].shape) == (128, 64)
    core = of3pair.TemplateEmbedderCore(64, 128, TEMPLATE_STACK_CFG, {"linear_t": {"bias": False, "init": "default"}})
    assert tuple(core.linear_t.weight.shape) == (128, 64) and core.linear_t.bias is None
    assert all(k.startswith("template_pair_stack.") or k == "linear_t.weight" for k in core.state_dict())
    sig = inspect.signature(of3pair.TemplatePairStack.forward)
    for name in ("t", "mask", "chunk_size", "use_deepspeed_evo_attention", "use_cueq_triangle_kernels", "use_lma",
                 "inplace_safe", "_mask_trans"):
        assert name in sig.parameters
    with pytest.raises(ValueError):
        of3pair.TemplatePairStack(**dict(TEMPLATE_STACK_CFG, transition_type="relu"))


def _fake_model_state_dict():
    """Keys as a reference model's state dict spells them, random values."""
    gen = torch.Generator().manual_seed(5)
    sd = {}
    for i in range(2):
        blk = of3pair.PairBlock(128, 128, 32, 4, "swiglu", 4, 0.25, False, 1e9)
        for k, v in blk.state_dict().items():
            sd["pairformer_stack.blocks.%d.pair_stack.%s" % (i, k)] = torch.randn(v.shape, generator=gen)
        sd["pairformer_stack.blocks.%d.attn_pair_bias.layer_norm_z.weight" % i] = torch.randn(128, generator=gen)
        sd["pairformer_stack.blocks.%d.attn_pair_bias.layer_norm_z.bias" % i] = torch.randn(128, generator=gen)
        sd["pairformer_stack.blocks.%d.attn_pair_bias.linear_z.weight" % i] = torch.randn(16, 128, generator=gen)
        sd["pairformer_stack.blocks.%d.attn_pair_bias.mha.linear_q.weight" % i] = torch.randn(384, 384, generator=gen)
    core = of3pair.TemplateEmbedderCore(64, 128, TEMPLATE_STACK_CFG)
    for k, v in core.state_dict().items():
        sd["template_embedder." + k] = torch.randn(v.shape, generator=gen)
    sd["template_embedder.template_pair_embedder.linear_z.weight"] = torch.randn(64, 128, generator=gen)
    return sd


@pytest.mark.parametrize("container", ["pretrained", "lightning", "deepspeed", "ema"])
def test_checkpoint_slices_load_into_the_modules(container):
    from of3pair import checkpoint as ck

    raw = _fake_model_state_dict()
    if container == "pretrained":
        ckpt = raw
    elif container == "lightning":
        ckpt = {"state_dict": {"model." + k: v for k, v in raw.items()}, "epoch": 3}
    elif container == "deepspeed":
        ckpt = {"module": {"model." + k: v for k, v in raw.items()}}
    else:
        ckpt = {"state_dict": {"model." + k: torch.zeros_like(v) for k, v in raw.items()}, "ema": {"params": raw}}
    sd = ck.state_dict_from_checkpoint(ckpt, init_from_ema_weights=(container == "ema"))
    assert all(k.startswith("model.") for k in sd)
    assert ck.pairformer_block_count(sd) == 2
    blocks = [of3pair.PairBlock(128, 128, 32, 4, "swiglu", 4, 0.25, False, 1e9) for _ in range(2)]
    ck.load_pairformer_pair_blocks(blocks, sd)
    assert torch.equal(blocks[1].tri_att_end.mha.linear_o.weight,
                       raw["pairformer_stack.blocks.1.pair_stack.tri_att_end.mha.linear_o.weight"])
    assert torch.equal(blocks[0].pair_transition.swiglu.linear_a.weight,
                       raw["pairformer_stack.blocks.0.pair_stack.pair_transition.swiglu.linear_a.weight"])
    core = ck.load_template_embedder(of3pair.TemplateEmbedderCore(64, 128, TEMPLATE_STACK_CFG), sd)
    assert torch.equal(core.linear_t.weight, raw["template_embedder.linear_t.weight"])
    assert torch.equal(core.template_pair_stack.layer_norm.bias, raw["template_embedder.template_pair_stack.layer_norm.bias"])
    proj = ck.load_pair_bias_projection(of3pair.PairBiasProjection(128, 16), sd,
                                        "model.pairformer_stack.blocks.1.attn_pair_bias.")
    assert torch.equal(proj.linear_z.weight, raw["pairformer_stack.blocks.1.attn_pair_bias.linear_z.weight"])


def test_checkpoint_loading_reports_missing_and_unexpected_keys(tmp_path):
    from of3pair import checkpoint as ck

    sd = {"model." + k: v for k, v in _fake_model_state_dict().items()}
    blk = of3pair.PairBlock(128, 128, 32, 4, "swiglu", 4, 0.25, False, 1e9)
    with pytest.raises(KeyError):
        ck.load_pair_block(blk, sd, "model.pairformer_stack.blocks.7.pair_stack.")
    broken = dict(sd)
    del broken["model.pairformer_stack.blocks.0.pair_stack.tri_mul_in.linear_g.weight"]
    with pytest.raises(KeyError, match="linear_g"):
        ck.load_pair_block(blk, broken, "model.pairformer_stack.blocks.0.pair_stack.")
    extra = dict(sd)
    extra["model.template_embedder.linear_u.weight"] = torch.zeros(1)
    with pytest.raises(KeyError, match="linear_u"):
        ck.load_template_embedder(of3pair.TemplateEmbedderCore(64, 128, TEMPLATE_STACK_CFG), extra)
    # files are read with the loader that executes nothing
    path = tmp_path / "w.pt"
    torch.save({k[len("model."):]: v for k, v in sd.items()}, path)
    loaded = ck.state_dict_from_checkpoint(ck.load_checkpoint_file(path))
    assert sorted(loaded) == sorted(sd)


def test_pairformer_modules_take_the_reference_config_and_names():
    """architecture.pairformer of the reference's model config (model_config.py:268-287) constructs
    the stack; parameter names are the reference's."""
    cfg = dict(c_s=384, c_z=128, c_hidden_pair_bias=24, no_heads_pair_bias=16, c_hidden_mul=128,
               c_hidden_pair_att=32, no_heads_pair=4, no_blocks=3, transition_type="swiglu", transition_n=4,
               pair_dropout=0.25, fuse_projection_weights=False, blocks_per_ckpt=None, inf=1e9, use_reentrant=False,
               clear_cache_between_blocks=False, tune_chunk_size=False)
    stack = of3pair.PairFormerStack(**cfg)
    names = set(stack.state_dict())
    assert len(stack.blocks) == 3
    for k in ("pair_stack.tri_mul_out.linear_a_p.weight", "pair_stack.tri_att_end.mha.linear_o.weight",
              "pair_stack.pair_transition.swiglu.linear_a.weight", "attn_pair_bias.layer_norm_a.weight",
              "attn_pair_bias.layer_norm_z.bias", "attn_pair_bias.linear_z.weight", "attn_pair_bias.mha.linear_q.weight",
              "attn_pair_bias.mha.linear_q.bias", "attn_pair_bias.mha.linear_g.weight",
              "single_transition.layer_norm.weight", "single_transition.swiglu.linear_b.weight",
              "single_transition.linear_out.weight"):
        assert "blocks.2." + k in names
    sd = stack.state_dict()
    assert tuple(sd["blocks.0.attn_pair_bias.mha.linear_q.weight"].shape) == (384, 384)
    assert tuple(sd["blocks.0.attn_pair_bias.linear_z.weight"].shape) == (16, 128)
    assert tuple(sd["blocks.0.single_transition.swiglu.linear_a.weight"].shape) == (1536, 384)
    assert not any(k.endswith("mha.linear_k.bias") for k in names)
    sig = inspect.signature(of3pair.PairFormerStack.forward)
    for name in ("s", "z", "single_mask", "pair_mask", "chunk_size", "inplace_safe", "_mask_trans"):
        assert name in sig.parameters
    with pytest.raises(ValueError):
        of3pair.AttentionPairBias(384, 384, 384, 384, 128, 24, 16, use_ada_layer_norm=True)


def test_whole_pairformer_stack_loads_from_a_model_state_dict():
    from of3pair import checkpoint as ck

    cfg = dict(c_s=384, c_z=128, c_hidden_pair_bias=24, no_heads_pair_bias=16, c_hidden_mul=128,
               c_hidden_pair_att=32, no_heads_pair=4, no_blocks=2, transition_type="swiglu", transition_n=4,
               pair_dropout=0.25, fuse_projection_weights=False, blocks_per_ckpt=None, inf=1e9)
    src = of3pair.PairFormerStack(**cfg)
    gen = torch.Generator().manual_seed(9)
    sd = {"model.pairformer_stack." + k: torch.randn(v.shape, generator=gen) for k, v in src.state_dict().items()}
    sd["model.msa_module.blocks.0.linear.weight"] = torch.zeros(1)
    dst = ck.load_pairformer_stack(of3pair.PairFormerStack(**cfg), sd)
    for k, v in dst.state_dict().items():
        assert torch.equal(v, sd["model.pairformer_stack." + k])
    with pytest.raises(KeyError):
        ck.load_pairformer_stack(of3pair.PairFormerStack(**dict(cfg, no_blocks=3)), sd)


def test_modules_refuse_training_mode_and_inputs_that_want_gradients():
    """The kernels are the inference forward pass: no dropout, no autograd.  A module left in training
    mode (where the reference would apply pair_dropout and record gradients) or an input that requires
    a gradient must raise instead of silently returning an un-dropped, non-differentiable result."""
    blk = of3pair.PairBlock(64, 64, 16, 4, "swiglu", 2, 0.25, False, 1e9)
    z = torch.zeros(1, 8, 8, 64)
    mask = torch.ones(1, 8, 8)
    assert blk.training
    with pytest.raises(RuntimeError, match="forward-only"):
        blk(z, mask)
    with torch.no_grad(), pytest.raises(RuntimeError, match="forward-only"):
        blk(z, mask)  # train mode without autograd would still skip the dropout
    blk.eval()
    with pytest.raises(RuntimeError, match="requires a gradient"):
        blk(z.clone().requires_grad_(True), mask)
    for m in (of3pair.TriangleMultiplicationOutgoing(64, 64), of3pair.TriangleAttention(64, 16, 4),
              of3pair.SwiGLUTransition(64, 2), of3pair.PairBiasProjection(64, 16)):
        with pytest.raises(RuntimeError, match="forward-only"):
            m(z) if isinstance(m, of3pair.PairBiasProjection) else m(z, mask)
    # in eval mode the only refusal left is the missing device (no CPU path)
    with pytest.raises(RuntimeError, match="GPU"):
        blk(z, mask)


def test_build_stamp_detects_edited_sources(tmp_path, monkeypatch):
    """is_built() is more than a file-exists test: the digest written at build time must match the
    sources as they are now, and the loader refuses a library whose sources changed."""
    from of3pair import build as B

    lib = tmp_path / "libof3pair.so"
    stamp = tmp_path / "libof3pair.sources.sha256"
    monkeypatch.setattr(B, "LIB_PATH", str(lib))
    monkeypatch.setattr(B, "STAMP_PATH", str(stamp))
    assert not B.is_built() and not B.is_stale()
    lib.write_bytes(b"\x7fELF")
    assert B.is_built()  # no stamp: cannot be judged, accepted
    stamp.write_text(B.source_digest() + "\n")
    assert B.is_built() and not B.is_stale()
    stamp.write_text("0" * 64 + "\n")
    assert B.is_stale() and not B.is_built()


def test_fused_trimul_state_dict_names_and_pair_block_switch():
    """fuse_projection_weights=True builds the reference's FusedTriangleMultiplication modules
    (base_blocks.py:260-266; keys linear_ab_p / linear_ab_g with stacked [2 * c_hidden, c_z] weights)."""
    m = of3pair.FusedTriangleMultiplicationOutgoing(128, 128)
    want = {
        "layer_norm_in.weight": (128,), "layer_norm_in.bias": (128,),
        "layer_norm_out.weight": (128,), "layer_norm_out.bias": (128,),
        "linear_ab_p.weight": (256, 128), "linear_ab_g.weight": (256, 128),
        "linear_g.weight": (128, 128), "linear_z.weight": (128, 128),
    }
    assert {k: tuple(v.shape) for k, v in m.state_dict().items()} == want
    assert m._outgoing and not of3pair.FusedTriangleMultiplicationIncoming(64, 64)._outgoing
    assert m.linear_ab_g.weight.abs().max() == 0 and m.linear_z.weight.abs().max() == 0 and m.linear_ab_p.weight.std() > 0
    w = m._weights()
    assert w[4].data_ptr() == m.linear_ab_p.weight.data_ptr() and w[4].shape == (128, 128) and w[4].is_contiguous()
    assert w[6].data_ptr() == m.linear_ab_p.weight[128:].data_ptr() and w[6].is_contiguous()
    blk = of3pair.PairBlock(64, 64, 16, 4, "swiglu", 2, 0.0, True, 1e9)
    assert isinstance(blk.tri_mul_out, of3pair.FusedTriangleMultiplicationOutgoing)
    assert isinstance(blk.tri_mul_in, of3pair.FusedTriangleMultiplicationIncoming)
    assert "tri_mul_in.linear_ab_g.weight" in blk.state_dict()
    with pytest.raises(ValueError):  # the kernels have no bias term
        of3pair.FusedTriangleMultiplicationOutgoing(64, 64, linear_init_params={"linear_ab_p": {"bias": True, "init": "default"}})
    with pytest.raises(NotImplementedError):  # tmu.py:612-618
        m.eval()(torch.zeros(1, 4, 4, 128), use_cueq_triangle_kernels=True)

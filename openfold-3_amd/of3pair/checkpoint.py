"""Loading reference checkpoints into the modules of this package.

The modules keep the reference's parameter names, so loading is a matter of cutting the right
slice out of a model state dict:

    model.pairformer_stack.*                              -> PairFormerStack      (model.py:95)
    model.pairformer_stack.blocks.<i>.pair_stack.*        -> PairBlock            (pairformer.py:91)
    model.template_embedder.template_pair_stack.*         -> TemplatePairStack    (template_module.py:395)
    model.template_embedder.linear_t.weight               -> TemplateEmbedderCore (template_module.py:403)
    ...attn_pair_bias.layer_norm_z / linear_z             -> PairBiasProjection   (attention_pair_bias.py:106-107)

Checkpoint containers follow openfold3/core/utils/checkpoint_loading_utils.py:55-72.  Files are
read with torch.load(weights_only=True): nothing in a checkpoint is executed.
"""
from __future__ import annotations

import re
from typing import Iterable, Mapping

import torch


def load_checkpoint_file(path) -> dict:
    """A single-file checkpoint (pre-trained weights, Lightning or EMA container) as a dict."""
    return torch.load(path, map_location="cpu", weights_only=True)


def state_dict_from_checkpoint(ckpt: Mapping, init_from_ema_weights: bool = False) -> dict:
    """checkpoint_loading_utils.py:55-72: pre-trained files hold the model's parameters without
    the "model." prefix; EMA weights live under ckpt["ema"]["params"]; DeepSpeed files under
    "module"; Lightning files under "state_dict".  The result always carries "model." keys."""
    pretrained = "module" not in ckpt and "state_dict" not in ckpt
    if pretrained:
        return {"model." + k: v for k, v in ckpt.items()}
    if init_from_ema_weights:
        return {"model." + k: v for k, v in ckpt["ema"]["params"].items()}
    if "module" in ckpt:
        return dict(ckpt["module"])
    return dict(ckpt["state_dict"])


def sub_state_dict(state_dict: Mapping, prefix: str) -> dict:
    """The entries under `prefix`, with the prefix removed."""
    return {k[len(prefix):]: v for k, v in state_dict.items() if k.startswith(prefix)}


def _load(module, sd: Mapping, what: str, allow_extra: Iterable[str] = ()):
    if not sd:
        raise KeyError("no parameters found for %s" % what)
    missing, unexpected = module.load_state_dict(sd, strict=False)
    unexpected = [k for k in unexpected if not any(k.startswith(p) for p in allow_extra)]
    if missing or unexpected:
        raise KeyError("%s: missing keys %s, unexpected keys %s" % (what, sorted(missing), sorted(unexpected)))
    return module


def load_pair_block(block, state_dict: Mapping, prefix: str):
    """One PairBlock from the keys under `prefix` (e.g. "model.pairformer_stack.blocks.0.pair_stack.")."""
    return _load(block, sub_state_dict(state_dict, prefix), prefix)


def pairformer_block_count(state_dict: Mapping, stack: str = "model.pairformer_stack.") -> int:
    pat = re.compile(re.escape(stack) + r"blocks\.(\d+)\.pair_stack\.")
    ids = {int(m.group(1)) for k in state_dict for m in [pat.match(k)] if m}
    return max(ids) + 1 if ids else 0


def load_pairformer_pair_blocks(blocks, state_dict: Mapping, stack: str = "model.pairformer_stack."):
    """blocks[i] <- <stack>blocks.<i>.pair_stack.* for every PairBlock of the list."""
    for i, blk in enumerate(blocks):
        load_pair_block(blk, state_dict, "%sblocks.%d.pair_stack." % (stack, i))
    return blocks


def load_pairformer_stack(stack, state_dict: Mapping, prefix: str = "model.pairformer_stack."):
    """PairFormerStack <- every key under `prefix` (blocks.<i>.pair_stack.*, .attn_pair_bias.*,
    .single_transition.*); the number of blocks must match."""
    return _load(stack, sub_state_dict(state_dict, prefix), prefix)


def load_template_embedder(core, state_dict: Mapping, prefix: str = "model.template_embedder."):
    """TemplateEmbedderCore <- template_pair_stack.* and linear_t.weight under `prefix`; the
    feature embedder's keys (template_pair_embedder.*) belong to no module here and are skipped."""
    return _load(core, sub_state_dict(state_dict, prefix), prefix, allow_extra=("template_pair_embedder.",))


def load_pair_bias_projection(proj, state_dict: Mapping, prefix: str):
    """PairBiasProjection <- layer_norm_z.* and linear_z.weight of the AttentionPairBias under
    `prefix` (e.g. "model.pairformer_stack.blocks.0.attn_pair_bias."); its other keys are skipped."""
    sd = {k: v for k, v in sub_state_dict(state_dict, prefix).items()
          if k.startswith("layer_norm_z.") or k.startswith("linear_z.")}
    return _load(proj, sd, prefix)

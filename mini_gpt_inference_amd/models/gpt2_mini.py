"""The GPT-2-style dense decoder of the reference (src/minigpt_infer/model.py:118-187) as data:
which parts each layer has, their constants, and the checkpoint names of their tensors.

Tensor names are the reference's state-dict names (model.py:43-44,96-97,107-110,123-128).
Fixed by the architecture's code rather than by config.json, and therefore set here and passed
to the parts as parameters: the MLP's hidden size 4*n_embd (model.py:96), GELU-tanh
(model.py:101), scale 1/sqrt(head_dim) (SDPA's default, model.py:87), pre-norm blocks
(model.py:112-115), learned absolute positions (model.py:124), a head tied to the token
embedding with no bias (model.py:128-130).
"""

from __future__ import annotations

import math
from typing import List, Tuple

from ..config.model_config import GPTConfig
from ..config.registry import Architecture, register_architecture
from ..parts.base import PartSpec
from ..parts.model import LayerRun, LayerSpec, ModelSpec

NAME = "gpt2-mini"
MLP_RATIO = 4   # src/minigpt_infer/model.py:96


def _w(prefix: str, has_bias: bool, /, **names: str) -> dict:
    """Parameter name -> checkpoint name, dropping the bias entries when the model has none."""
    return {local: prefix + name for local, name in names.items() if has_bias or not local.endswith("bias")}


def model_spec(cfg: GPTConfig) -> ModelSpec:
    c, d = cfg.n_embd, cfg.head_dim
    layers = []
    for i in range(cfg.n_layer):
        p = f"blocks.{i}."
        layers.append(LayerSpec(
            arrangement=PartSpec("pre_norm", {"width": c}),
            norm1=PartSpec("layer_norm", {"width": c, "eps": cfg.layer_norm_eps, "bias": cfg.bias},
                           _w(p + "ln1.", cfg.bias, weight="weight", bias="bias")),
            mixer=PartSpec("paged_causal_attention",
                           {"width": c, "n_head": cfg.n_head, "head_dim": d, "bias": cfg.bias,
                            "n_kv_head": cfg.n_head, "scale": 1.0 / math.sqrt(d), "window": 0},
                           _w(p + "attn.", cfg.bias, qkv_weight="qkv.weight", qkv_bias="qkv.bias",
                              proj_weight="proj.weight", proj_bias="proj.bias")),
            norm2=PartSpec("layer_norm", {"width": c, "eps": cfg.layer_norm_eps, "bias": cfg.bias},
                           _w(p + "ln2.", cfg.bias, weight="weight", bias="bias")),
            feed_forward=PartSpec("dense_mlp",
                                  {"width": c, "hidden": MLP_RATIO * c, "bias": cfg.bias,
                                   "activation": "gelu_tanh"},
                                  _w(p + "mlp.", cfg.bias, fc_weight="fc.weight", fc_bias="fc.bias",
                                     proj_weight="proj.weight", proj_bias="proj.bias")),
        ))
    return ModelSpec(
        width=c,
        vocab_size=cfg.vocab_size,
        embedding=PartSpec("token_embedding", {"vocab_size": cfg.vocab_size, "width": c},
                           {"weight": "tok_emb.weight"}),
        position=PartSpec("learned_absolute", {"max_positions": cfg.block_size, "width": c},
                          {"weight": "pos_emb.weight"}),
        layers=tuple(layers),
        order=tuple(LayerRun(i) for i in range(cfg.n_layer)),
        final_norm=PartSpec("layer_norm", {"width": c, "eps": cfg.layer_norm_eps, "bias": cfg.bias},
                            _w("ln_f.", cfg.bias, weight="weight", bias="bias")),
        head=PartSpec("linear_head", {"vocab_size": cfg.vocab_size, "width": c, "tied": True},
                      {"weight": "tok_emb.weight"}),
        max_positions=cfg.block_size,
        # a torch state dict lists the tied head a second time (model.py:128-130)
        tied_aliases=(("lm_head.weight", "tok_emb.weight"),),
    )


def init_plan(cfg: GPTConfig) -> List[Tuple[str, Tuple[int, ...], str, float]]:
    """Random-weights rule, in drawing order.  Matrices and tables N(0, 0.02), the two residual
    projections N(0, 0.02/sqrt(2*n_layer)) (reference: src/minigpt_infer/model.py:132-144).
    Where the reference sets biases to zero and LayerNorm gains to one, this mode draws biases
    N(0, 0.01) and gains 1 + N(0, 0.1), so that a fault in a bias or gain path shows."""
    c, f = cfg.n_embd, MLP_RATIO * cfg.n_embd
    std, res_std = 0.02, 0.02 / math.sqrt(2 * cfg.n_layer)
    plan: List[Tuple[str, Tuple[int, ...], str, float]] = [
        ("tok_emb.weight", (cfg.vocab_size, c), "normal", std),
        ("pos_emb.weight", (cfg.block_size, c), "normal", std),
    ]

    def norm(prefix: str) -> None:
        plan.append((prefix + "weight", (c,), "gain", 0.1))
        if cfg.bias:
            plan.append((prefix + "bias", (c,), "normal", 0.01))

    def lin(prefix: str, out: int, inn: int, s: float) -> None:
        plan.append((prefix + "weight", (out, inn), "normal", s))
        if cfg.bias:
            plan.append((prefix + "bias", (out,), "normal", 0.01))

    for i in range(cfg.n_layer):
        p = f"blocks.{i}."
        norm(p + "ln1.")
        lin(p + "attn.qkv.", 3 * c, c, std)
        lin(p + "attn.proj.", c, c, res_std)
        norm(p + "ln2.")
        lin(p + "mlp.fc.", f, c, std)
        lin(p + "mlp.proj.", c, f, res_std)
    norm("ln_f.")
    return plan


register_architecture(Architecture(NAME, GPTConfig.from_json_dict, model_spec, init_plan))

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
from dataclasses import asdict, dataclass, fields
from typing import Any, List, Mapping, Tuple

from ..config.model_config import ConfigError
from ..config.registry import Architecture, register_architecture
from ..parts.base import PartSpec
from ..parts.model import LayerRun, LayerSpec, ModelSpec

NAME = "gpt2-mini"
MLP_RATIO = 4   # src/minigpt_infer/model.py:96

# Keys a config.json may carry that the engine reads past: the reference forces dropout to 0 at
# inference (src/minigpt_infer/loader.py:58).
_IGNORED_KEYS = {"dropout", "model_type", "torch_dtype"}


@dataclass(frozen=True)
class GPTConfig:
    """The architecture's typed configuration, read from its own config.json keys: the fields of the
    reference's GPTConfig dataclass (src/minigpt_infer/config.py:10-18; model.py:118-130).
    layer_norm_eps is added because the reference leaves it at nn.LayerNorm's default
    (model.py:107,109,127) and a model folder has to be able to say otherwise."""

    architecture: str
    n_layer: int
    n_embd: int
    n_head: int
    vocab_size: int
    block_size: int          # rows of the learned position table = most positions
    bias: bool               # biases on every Linear and every LayerNorm
    layer_norm_eps: float = 1e-5

    def __post_init__(self) -> None:
        for name in ("n_layer", "n_embd", "n_head", "vocab_size", "block_size"):
            value = getattr(self, name)
            if not isinstance(value, int) or isinstance(value, bool) or value <= 0:
                raise ConfigError(f"{name} must be a positive integer, got {value!r}")
        if not isinstance(self.bias, bool):
            raise ConfigError(f"bias must be true or false, got {self.bias!r}")
        if not (isinstance(self.layer_norm_eps, float) and self.layer_norm_eps > 0.0):
            raise ConfigError(f"layer_norm_eps must be a positive float, got {self.layer_norm_eps!r}")
        # src/minigpt_infer/model.py:39
        if self.n_embd % self.n_head != 0:
            raise ConfigError(
                f"n_embd ({self.n_embd}) is not divisible by n_head ({self.n_head})"
            )

    @property
    def head_dim(self) -> int:
        return self.n_embd // self.n_head

    def to_json_dict(self) -> dict[str, Any]:
        return asdict(self)

    @classmethod
    def from_json_dict(cls, raw: Mapping[str, Any]) -> "GPTConfig":
        known = {f.name for f in fields(cls)}
        data = dict(raw)
        if "architecture" not in data and "model_type" in data:
            data["architecture"] = data["model_type"]
        unknown = sorted(k for k in data if k not in known and k not in _IGNORED_KEYS
                         and not k.startswith("_"))
        if unknown:
            raise ConfigError(f"config.json has keys this architecture does not know: {unknown}")
        required = [f.name for f in fields(cls) if f.name != "layer_norm_eps"]
        missing = [k for k in required if k not in data]
        if missing:
            raise ConfigError(f"config.json lacks required keys: {missing}")
        kwargs = {k: data[k] for k in known if k in data}
        if "layer_norm_eps" in kwargs:
            kwargs["layer_norm_eps"] = float(kwargs["layer_norm_eps"])
        return cls(**kwargs)


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


register_architecture(Architecture(NAME, GPTConfig.from_json_dict, model_spec, init_plan, GPTConfig.to_json_dict))

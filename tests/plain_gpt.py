"""A plain, slow implementation of the GPT-2-style decoder, written from the reference's
formulas.  Whole sequences, no cache, one function per part, float64 throughout, no code
shared with the engine.  Everything the engine computes is compared with this.

Citations are file:line into the reference repository.
"""

from __future__ import annotations

import json
import math
import os
from typing import Dict, List, Optional, Sequence

import numpy as np
import torch
from safetensors import safe_open

DT = torch.float64


# ----------------------------------------------------------------------------- parts
def plain_layer_norm(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], eps: float) -> torch.Tensor:
    """nn.LayerNorm over the last dim: (x - mean) / sqrt(biased var + eps) * weight + bias
    (src/minigpt_infer/model.py:107,109,127)."""
    mean = x.mean(dim=-1, keepdim=True)
    var = ((x - mean) ** 2).mean(dim=-1, keepdim=True)
    y = (x - mean) / torch.sqrt(var + eps) * weight
    return y + bias if bias is not None else y


def plain_gelu_tanh(u: torch.Tensor) -> torch.Tensor:
    """F.gelu(u, approximate="tanh") (src/minigpt_infer/model.py:101):
    0.5 u (1 + tanh(sqrt(2/pi) (u + 0.044715 u^3)))."""
    return 0.5 * u * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (u + 0.044715 * u ** 3)))


def plain_linear(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor]) -> torch.Tensor:
    """nn.Linear: y = x W^T + b with W stored [out, in] (src/minigpt_infer/model.py:43-44,96-97)."""
    y = x @ weight.t()
    return y + bias if bias is not None else y


def plain_split_heads(qkv: torch.Tensor, n_head: int, n_kv_head: Optional[int] = None):
    """q, k, v = split of the fused projection; head i = columns i*D..(i+1)*D
    (src/minigpt_infer/model.py:49-53).  Returns [H, T, D] each ([Hkv, T, D] for k and v)."""
    n_kv_head = n_kv_head or n_head
    t = qkv.shape[0]
    d = qkv.shape[1] // (n_head + 2 * n_kv_head)
    q, k, v = qkv.split([n_head * d, n_kv_head * d, n_kv_head * d], dim=1)
    return (q.view(t, n_head, d).transpose(0, 1), k.view(t, n_kv_head, d).transpose(0, 1),
            v.view(t, n_kv_head, d).transpose(0, 1))


def plain_causal_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: Optional[float] = None,
                           window: int = 0, causal: bool = True) -> torch.Tensor:
    """softmax(q k^T * scale + mask) v per head, scale 1/sqrt(D) by default; query t sees keys
    0..t (is_causal=True of src/minigpt_infer/model.py:72,87 for a whole prompt), with a window only
    the last `window` of them.  q: [H, T, D], k, v: [Hkv, T, D].  Returns [T, H*D], heads
    concatenated head-major (src/minigpt_infer/model.py:89)."""
    h, t, d = q.shape
    hk = k.shape[0]
    if scale is None:
        scale = 1.0 / math.sqrt(d)
    rep = h // hk
    out = torch.empty(t, h * d, dtype=q.dtype)
    pos = torch.arange(t)
    allowed = torch.ones(t, t, dtype=torch.bool)
    if causal:
        allowed = pos[None, :] <= pos[:, None]
        if window > 0:
            allowed &= pos[None, :] > pos[:, None] - window
    for i in range(h):
        s = (q[i] @ k[i // rep].t()) * scale
        s = s.masked_fill(~allowed, float("-inf"))
        p = torch.softmax(s, dim=-1)
        out[:, i * d:(i + 1) * d] = p @ v[i // rep]
    return out


def plain_embed(ids: torch.Tensor, tok_emb: torch.Tensor, pos_emb: Optional[torch.Tensor],
                first_position: int = 0) -> torch.Tensor:
    """x0[t] = tok_emb[id_t] + pos_emb[t] (src/minigpt_infer/model.py:183; reference.py:109-110)."""
    x = tok_emb[ids]
    if pos_emb is not None:
        x = x + pos_emb[first_position:first_position + ids.shape[0]]
    return x


def plain_attention_layer(h: torch.Tensor, w: Dict[str, torch.Tensor], prefix: str, n_head: int) -> torch.Tensor:
    """CausalSelfAttention.forward without a cache (src/minigpt_infer/reference.py:38-50)."""
    qkv = plain_linear(h, w[prefix + "qkv.weight"], w.get(prefix + "qkv.bias"))
    q, k, v = plain_split_heads(qkv, n_head)
    y = plain_causal_attention(q, k, v)
    return plain_linear(y, w[prefix + "proj.weight"], w.get(prefix + "proj.bias"))


def plain_mlp(h: torch.Tensor, w: Dict[str, torch.Tensor], prefix: str) -> torch.Tensor:
    """proj(gelu_tanh(fc(x))) (src/minigpt_infer/model.py:100-101)."""
    u = plain_linear(h, w[prefix + "fc.weight"], w.get(prefix + "fc.bias"))
    return plain_linear(plain_gelu_tanh(u), w[prefix + "proj.weight"], w.get(prefix + "proj.bias"))


def plain_block(x: torch.Tensor, w: Dict[str, torch.Tensor], prefix: str, n_head: int, eps: float) -> torch.Tensor:
    """x = x + attn(ln1(x)); x = x + mlp(ln2(x)) (src/minigpt_infer/model.py:112-115)."""
    x = x + plain_attention_layer(plain_layer_norm(x, w[prefix + "ln1.weight"], w.get(prefix + "ln1.bias"), eps),
                                  w, prefix + "attn.", n_head)
    x = x + plain_mlp(plain_layer_norm(x, w[prefix + "ln2.weight"], w.get(prefix + "ln2.bias"), eps),
                      w, prefix + "mlp.")
    return x


def plain_forward(w: Dict[str, torch.Tensor], cfg: dict, ids: Sequence[int],
                  rows: Optional[Sequence[int]] = None) -> torch.Tensor:
    """Whole-sequence forward, logits at every position [T, V], or at the positions `rows` only
    (src/minigpt_infer/reference.py:105-114; tied head: reference.py:89-90)."""
    ids_t = torch.as_tensor(list(ids), dtype=torch.long)
    if ids_t.numel() > cfg["block_size"]:
        raise ValueError(f"sequence length {ids_t.numel()} > block_size {cfg['block_size']}")
    eps = float(cfg.get("layer_norm_eps", 1e-5))
    x = plain_embed(ids_t, w["tok_emb.weight"], w["pos_emb.weight"])
    for layer in range(cfg["n_layer"]):
        x = plain_block(x, w, f"blocks.{layer}.", cfg["n_head"], eps)
    x = plain_layer_norm(x, w["ln_f.weight"], w.get("ln_f.bias"), eps)
    if rows is not None:
        x = x[list(rows)]
    return x @ w["tok_emb.weight"].t()


# ----------------------------------------------------------------------------- weights
def read_model_folder(model_dir: str):
    """(config dict, tensors as float64) straight from the files."""
    with open(os.path.join(model_dir, "config.json")) as fh:
        cfg = json.load(fh)
    w: Dict[str, torch.Tensor] = {}
    with safe_open(os.path.join(model_dir, "model.safetensors"), framework="pt", device="cpu") as fh:
        for name in fh.keys():
            w[name] = fh.get_tensor(name).to(DT)
    return cfg, w


# ----------------------------------------------------------------------------- sampling
_M64 = (1 << 64) - 1


def _mix64(z: int) -> int:
    z ^= z >> 30
    z = (z * 0xBF58476D1CE4E5B9) & _M64
    z ^= z >> 27
    z = (z * 0x94D049BB133111EB) & _M64
    z ^= z >> 31
    return z


def plain_uniform(engine_seed: int, request_seed: int, index: int) -> float:
    """The engine's counter-based uniform number in [0, 1): a function of (engine seed, request
    seed, index of the output token) only.  Not in the reference, which draws from one shared
    torch generator (src/minigpt_infer/sampling.py:131-132)."""
    z = ((engine_seed & _M64) * 0x9E3779B97F4A7C15 + (request_seed & _M64) * 0xD1B54A32D192ED03
         + (index & _M64) * 0x8CB92BA72F3D8DD7 + 0x2545F4914F6CDD1D) & _M64
    z = _mix64(_mix64(z))
    return (z >> 40) / 16777216.0


def plain_top_k_mask(scaled: np.ndarray, k: int) -> np.ndarray:
    """Keep values >= the k-th largest; ties pass; k clamped to [1, V]
    (src/minigpt_infer/sampling.py:39-52)."""
    k = max(1, min(int(k), scaled.size))
    threshold = np.sort(scaled)[::-1][k - 1]
    return scaled >= threshold


def plain_top_p_mask(scaled: np.ndarray, keep: np.ndarray, p: float) -> np.ndarray:
    """Sort descending, softmax, drop a token iff the mass strictly before it exceeds p; the first
    always stays (src/minigpt_infer/sampling.py:55-76).  Written per value: a token stays iff the
    mass of the strictly larger kept ones is <= p (equal to the reference's rule when values
    are distinct; equal values stay or go together)."""
    vals = np.where(keep, scaled, -np.inf)
    w = np.exp(vals - vals.max())
    z = w.sum()
    order = np.argsort(-vals, kind="stable")
    out = np.zeros_like(keep)
    sorted_vals, sorted_w = vals[order], w[order]
    before = np.concatenate([[0.0], np.cumsum(sorted_w)[:-1]])
    # mass of strictly larger values: for runs of equal values use the run's first entry
    first_of_run = np.concatenate([[True], sorted_vals[1:] != sorted_vals[:-1]])
    run_start_mass = np.maximum.accumulate(np.where(first_of_run, before, 0.0))
    stay = (run_start_mass <= p * z) & np.isfinite(sorted_vals)
    out[order] = stay
    return out


def plain_sample(logits: np.ndarray, temperature: float, top_k: Optional[int], top_p: Optional[float],
                 u: float, real_vocab: Optional[int] = None):
    """Next token from float logits.  Order as the reference: vocabulary mask, temperature, top-k,
    top-p, softmax (src/minigpt_infer/sampling.py:116-130, src/minigpt_infer/engine/engine.py:154-156);
    temperature <= 0 is the argmax of the unscaled logits (sampling.py:134-136), lowest index on ties.
    The draw is by inverse CDF in vocabulary order with the given uniform number.  Returns
    (token, cdf_low, cdf_high, total): the chosen token's interval of the unnormalised CDF."""
    lg = np.asarray(logits, dtype=np.float64).copy()
    nv = lg.size if real_vocab is None else min(real_vocab, lg.size)
    lg[nv:] = -np.inf
    if temperature <= 0:
        return int(np.argmax(lg)), 0.0, 0.0, 0.0
    # the engine divides in float32
    scaled = (np.asarray(logits, dtype=np.float32) / np.float32(max(temperature, 1e-6))).astype(np.float64)
    scaled[nv:] = -np.inf
    keep = np.isfinite(scaled)
    if top_k is not None and top_k < nv:
        keep &= plain_top_k_mask(np.where(keep, scaled, -np.inf), top_k)
    if top_p is not None and top_p < 1.0:
        keep &= plain_top_p_mask(scaled, keep, top_p)
    w = np.where(keep, np.exp(scaled - scaled[keep].max()), 0.0)
    cdf = np.cumsum(w)
    total = cdf[-1]
    target = u * total
    idx = int(np.searchsorted(cdf, target, side="right"))
    kept_idx = np.nonzero(keep)[0]
    if idx >= lg.size:
        idx = int(kept_idx[-1])
    lo = cdf[idx - 1] if idx > 0 else 0.0
    return idx, float(lo), float(cdf[idx]), float(total)


def plain_greedy_generate(w: Dict[str, torch.Tensor], cfg: dict, prompt: Sequence[int], n_new: int,
                          real_vocab: Optional[int] = None) -> List[int]:
    """Full re-forward per token, argmax of the last position
    (src/minigpt_infer/reference.py:149-175)."""
    ids = list(prompt)
    for _ in range(n_new):
        logits = plain_forward(w, cfg, ids)[-1].numpy()
        tok, *_ = plain_sample(logits, 0.0, None, None, 0.0, real_vocab)
        ids.append(tok)
    return ids[len(prompt):]

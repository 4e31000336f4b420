"""Tiny configurations, model folders and tolerances shared by the tests."""

from __future__ import annotations

import os
from typing import Callable, Dict, Optional

import numpy as np
import torch
from safetensors.torch import save_file

from mini_gpt_inference_amd import GPTConfig
from mini_gpt_inference_amd.config.model_config import write_config_json
from mini_gpt_inference_amd.weights.random_init import random_tensors

# Two tiny configurations that differ in every size and option (layers, width, heads, head size,
# vocabulary, positions, bias, eps), plus a long-context one for far-key tests.
CONFIGS: Dict[str, GPTConfig] = {
    "A": GPTConfig("gpt2-mini", n_layer=2, n_embd=64, n_head=4, vocab_size=257, block_size=64, bias=True,
                   layer_norm_eps=1e-5),
    "B": GPTConfig("gpt2-mini", n_layer=3, n_embd=96, n_head=3, vocab_size=503, block_size=128, bias=False,
                   layer_norm_eps=1e-6),
    # head sizes that are no power of two (48, 80) and a width that is no multiple of 64
    "C": GPTConfig("gpt2-mini", n_layer=2, n_embd=144, n_head=3, vocab_size=131, block_size=96, bias=True,
                   layer_norm_eps=1e-4),
    "D": GPTConfig("gpt2-mini", n_layer=1, n_embd=80, n_head=1, vocab_size=77, block_size=200, bias=False,
                   layer_norm_eps=1e-5),
    # head sizes that are no multiple of 16 (40, 12) and widths that are none either: the
    # architecture takes any n_embd that n_head divides (src/minigpt_infer/model.py:39-41)
    "E": GPTConfig("gpt2-mini", n_layer=2, n_embd=40, n_head=1, vocab_size=99, block_size=72, bias=True,
                   layer_norm_eps=1e-5),
    "F": GPTConfig("gpt2-mini", n_layer=2, n_embd=36, n_head=3, vocab_size=150, block_size=80, bias=False,
                   layer_norm_eps=1e-6),
    "LONG": GPTConfig("gpt2-mini", n_layer=1, n_embd=48, n_head=1, vocab_size=61, block_size=640, bias=True,
                      layer_norm_eps=1e-3),
}
SEEDS = {"A": 0, "B": 1, "C": 3, "D": 4, "E": 5, "F": 6, "LONG": 2}
# The init rule's standard deviations give nearly uniform attention and tiny logits, which hides
# faults; the tests scale them up so that softmax is peaked and every path carries signal.
STD_SCALE = {"A": 5.0, "B": 5.0, "C": 4.0, "D": 5.0, "E": 6.0, "F": 6.0, "LONG": 6.0}

# Tolerances, fixed before any kernel was measured.  float32: summation order only.  bfloat16:
# activations and weights carry 8 bits of mantissa (relative 2^-9 per rounding, a handful of
# roundings per layer), the reference's own half-precision bound is 2e-2 (tests/test_triton.py:101).
TOL = {"float32": 2e-5, "bfloat16": 2e-2}


def write_model(path: str, name: str, edit: Optional[Callable[[Dict[str, torch.Tensor]], None]] = None,
                dtype: torch.dtype = torch.bfloat16) -> str:
    cfg = CONFIGS[name]
    tensors = random_tensors(cfg, SEEDS[name], dtype, STD_SCALE[name])
    if edit is not None:
        edit(tensors)
    os.makedirs(path, exist_ok=True)
    write_config_json(path, cfg)
    save_file({k: v.contiguous() for k, v in tensors.items()}, os.path.join(path, "model.safetensors"))
    return path


def assert_close(got, want, dtype: str, what: str = "") -> None:
    """max |got - want| <= TOL[dtype] * max(1, max |want|)."""
    got = got.detach().cpu().double() if isinstance(got, torch.Tensor) else torch.as_tensor(np.asarray(got)).double()
    want = (want.detach().cpu().double() if isinstance(want, torch.Tensor)
            else torch.as_tensor(np.asarray(want)).double())
    assert got.shape == want.shape, f"{what}: shape {tuple(got.shape)} vs {tuple(want.shape)}"
    assert torch.isfinite(got).all(), f"{what}: non-finite values in the engine's result"
    scale = max(1.0, float(want.abs().max()))
    err = float((got - want).abs().max())
    assert err <= TOL[dtype] * scale, f"{what}: max error {err:.3e} > {TOL[dtype]:.0e} * {scale:.3g}"


def random_ids(rng: np.random.Generator, vocab: int, n: int):
    return rng.integers(0, vocab, n).tolist()


# ----------------------------------------------------------------------------- trace plans
class TracePlan:
    """Steps of a trace in bin/trace_run's JSON form, plus the bookkeeping to put the logits that
    come back into one [length, vocab] array per request."""

    def __init__(self) -> None:
        self.steps = []        # JSON records
        self.wanted = {}       # step -> [(request, position)] in file order
        self._fed = {}         # request -> tokens fed so far
        self._live = {}        # request -> final length (for the pool size)
        self.max_tokens = 64
        self._live_history = []   # per step: final lengths of the requests live during it

    def add_step(self, entries, end=()):
        """entries: [(request id, tokens, final length of the request)]; every position is wanted."""
        step = len(self.steps)
        rec = {"step": step, "entries": [], "end": list(end)}
        rows = []
        for rid, toks, final_len in entries:
            start = self._fed.get(rid, 0)
            self._live[rid] = final_len
            rec["entries"].append({"id": rid, "tokens": list(toks), "want": list(range(len(toks)))})
            rows += [(rid, start + i) for i in range(len(toks))]
            self._fed[rid] = start + len(toks)
        self.max_tokens = max(self.max_tokens, sum(-(-n // 64) * 64 for n in self._live.values()))
        self._live_history.append(list(self._live.values()))
        for rid in end:
            self._live.pop(rid, None)
        self.steps.append(rec)
        self.wanted[step] = rows

    def tight_tokens(self, page_size):
        """The smallest pool, in tokens, that holds the live requests of every step."""
        return max(sum(-(-n // page_size) * page_size for n in lens) for lens in self._live_history)

    def assemble(self, outputs, lengths, vocab):
        """outputs: step -> array [wanted, vocab].  Returns request -> [length, vocab]."""
        res = {rid: np.full((n, vocab), np.nan, dtype=np.float64) for rid, n in lengths.items()}
        for step, rows in self.wanted.items():
            out = np.asarray(outputs[step], dtype=np.float64).reshape(len(rows), vocab)
            for (rid, pos), row in zip(rows, out):
                res[rid][pos] = row
        return res


def plan_whole(reqs):
    """Each request alone and whole, in one step."""
    plan = TracePlan()
    for rid, ids in reqs.items():
        plan.add_step([(rid, ids, len(ids))], end=[rid])
    return plan


def plan_tail(reqs, tail=32):
    """Most of it in one step, the last `tail` tokens one by one."""
    plan = TracePlan()
    for rid, ids in reqs.items():
        head = max(len(ids) - tail, 0)
        if head:
            plan.add_step([(rid, ids[:head], len(ids))])
        for i in range(head, len(ids)):
            plan.add_step([(rid, ids[i:i + 1], len(ids))], end=[rid] if i == len(ids) - 1 else [])
    return plan


def plan_portions(reqs, rng):
    """Portions of changing size, down to two tokens."""
    plan = TracePlan()
    sizes = [2, 7, 3, 16, 2, 5, 17, 33, 4]
    k = 0
    for rid, ids in reqs.items():
        pos = 0
        while pos < len(ids):
            q = min(sizes[k % len(sizes)], len(ids) - pos)
            k += 1
            plan.add_step([(rid, ids[pos:pos + q], len(ids))], end=[rid] if pos + q == len(ids) else [])
            pos += q
    return plan


def plan_mixed(reqs, rng, max_live=4, tail=32):
    """Up to max_live live requests: portions of some beside single decoded tokens of others; a
    request is now and then left out of a step; finished ones give their pages to later ones."""
    plan = TracePlan()
    queue = list(reqs.items())
    live = {}     # rid -> position
    while queue or live:
        while queue and len(live) < max_live:
            rid, _ = queue.pop(0)
            live[rid] = 0
        entries, end = [], []
        for rid in list(live):
            ids, pos = reqs[rid], live[rid]
            if len(live) > 1 and rng.random() < 0.2:
                continue       # left out of this step
            remaining = len(ids) - pos
            q = 1 if remaining <= tail else int(min(remaining - tail, rng.integers(2, 14)))
            entries.append((rid, ids[pos:pos + q], len(ids)))
            live[rid] = pos + q
            if live[rid] == len(ids):
                end.append(rid)
                del live[rid]
        if entries:
            plan.add_step(entries, end)
    return plan


PLANS = {"whole": lambda reqs, rng: plan_whole(reqs), "tail": lambda reqs, rng: plan_tail(reqs),
         "portions": plan_portions, "mixed": plan_mixed}


def run_plan_in_process(replayer, plan):
    outputs = {}
    for rec in plan.steps:
        logits = replayer.run_step(rec)
        if logits is not None:
            outputs[rec["step"]] = logits.cpu().numpy()
    return outputs

"""Trace replay: given token ids go through the engine's model, step function, cache manager and
kernels step by step; logits come back.  Nothing is sampled.  bin/trace_run is the command
line around this class.  The reference has no such tool; its tests drive model(ForwardBatch)
by hand (tests/test_cache.py:121-137)."""

from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..cache.kv_store import KVStore
from ..cache.manager import CacheManager, GroupGeometry
from ..weights.loader import load_model
from .step import ModelRunner

PAGE_SIZE = 16   # tokens per cache page; divides the 64-token rounding of max_tokens
MAX_LIVE = 8     # request slots


class TraceError(RuntimeError):
    pass


class TraceReplayer:
    def __init__(self, model_dir: str, dtype: str, max_tokens: int, device: str = "cuda:0",
                 page_size: int = PAGE_SIZE, max_live: int = MAX_LIVE, poison: bool = False) -> None:
        if dtype not in ("bfloat16", "float32"):
            raise TraceError("dtype must be bfloat16 or float32")
        self.device = torch.device(device)
        self.model, self.config, _ = load_model(model_dir, dtype, device)
        self.dtype = torch.bfloat16 if dtype == "bfloat16" else torch.float32
        self.page_size = page_size
        self.num_pages = max(1, -(-int(max_tokens) // page_size))
        layout = self.model.cache_layout
        geometry = [GroupGeometry(page_size, self.num_pages, g.window) for g in layout.groups]
        self.cache = CacheManager(geometry, max_live)
        self.store = KVStore(layout, geometry, max_live, self.dtype, self.device, poison=poison)
        self.runner = ModelRunner(self.model, self.cache, self.store, self.dtype, self.device,
                                  self.model.spec.max_positions)
        self.live: Dict[str, List[int]] = {}   # request id -> [cache slot, tokens cached]

    def run_step(self, record: dict) -> Optional[torch.Tensor]:
        """One line of a trace.  Returns float32 logits [wanted, vocab] on the device, or None when
        the step wants none.  The result lives in the step function's workspace: the next step
        overwrites it, so copy what is to be kept."""
        step = record.get("step")
        slots, ctx_lens, q_lens, tokens, rows, ids = [], [], [], [], [], []
        for entry in record.get("entries", []):
            toks = [int(t) for t in entry["tokens"]]
            if not toks:
                continue
            rid = entry["id"]
            if rid in ids:
                raise TraceError(f"step {step}: request {rid!r} appears twice")
            if rid not in self.live:
                slot = self.cache.acquire_slot()
                if slot < 0:
                    raise TraceError(f"step {step}: more live requests than the {self.cache.max_requests} slots")
                self.live[rid] = [slot, 0]
            slot, cached = self.live[rid]
            self.runner.check_positions([cached], [len(toks)])
            if not self.cache.reserve(slot, cached + len(toks)):
                raise TraceError(f"step {step}: request {rid!r} needs cache for {cached + len(toks)} tokens, "
                                 f"but the pool of {self.num_pages} pages of {self.page_size} tokens is used up")
            base = len(tokens)
            for w in entry.get("want", []):
                if not (0 <= int(w) < len(toks)):
                    raise TraceError(f"step {step}: want {w} lies outside the entry's {len(toks)} tokens")
                rows.append(base + int(w))
            ids.append(rid)
            slots.append(slot)
            ctx_lens.append(cached)
            q_lens.append(len(toks))
            tokens.extend(toks)
        logits = None
        if slots:
            logits = self.runner.step(slots, ctx_lens, q_lens, tokens, rows)
            for rid, q in zip(ids, q_lens):
                self.live[rid][1] += q
                self.cache.release_passed(*self.live[rid])
        for rid in record.get("end", []):
            if rid in self.live:
                self.cache.free_slot(self.live.pop(rid)[0])
        return logits if rows else None

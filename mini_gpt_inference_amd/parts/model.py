"""A decoder as data (ModelSpec) and the object that runs it (DecoderModel).

The specification lists the distinct layers and, separately, the order in which
they run.  The order is a list of runs; a run names a layer and says where its
mixer keeps its cache: in a cache of its own, or in the one an earlier run of
the same step writes (then it only reads).  A layer may appear in several runs.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Mapping, Optional, Tuple

import torch

from ..ops import residual
from ..ops.linear import LazyNorm
from . import block as _block  # noqa: F401  (registers the parts)
from . import embedding as _embedding  # noqa: F401
from . import feedforward as _feedforward  # noqa: F401
from . import mixers as _mixers  # noqa: F401
from . import norms as _norms  # noqa: F401
from . import positions as _positions  # noqa: F401
from .base import (ARRANGEMENTS, CacheBinding, EMBEDDINGS, FEED_FORWARDS, HEADS, KVNeed, MIXERS, NORMS,
                   POSITIONS, Part, PartSpec, StateNeed, StepContext, WeightRequest)


# categories of a layer's parts, and the registry of each
_LAYER_REGISTRIES = {"norm": NORMS, "mixer": MIXERS, "feed_forward": FEED_FORWARDS}


class LayerSpec:
    """A layer: an arrangement and the parts it arranges, each under a role name.

    parts: role -> (category, PartSpec) with category "norm", "mixer" or "feed_forward"; which
    roles there are is the arrangement's business (a pre-norm block has norm1, mixer, norm2,
    feed_forward; a block with one norm or two mixers has other roles).  The four roles of the
    pre-norm block can be given by keyword, or in that order."""

    def __init__(self, arrangement: PartSpec, norm1: Optional[PartSpec] = None, mixer: Optional[PartSpec] = None,
                 norm2: Optional[PartSpec] = None, feed_forward: Optional[PartSpec] = None, *,
                 parts: Optional[Mapping[str, Tuple[str, PartSpec]]] = None) -> None:
        named: Dict[str, Tuple[str, PartSpec]] = {}
        for role, (category, spec) in (parts or {}).items():
            if category not in _LAYER_REGISTRIES:
                raise ValueError(f"part {role!r}: category {category!r} is none of {sorted(_LAYER_REGISTRIES)}")
            named[role] = (category, spec)
        for role, category, spec in (("norm1", "norm", norm1), ("mixer", "mixer", mixer), ("norm2", "norm", norm2),
                                     ("feed_forward", "feed_forward", feed_forward)):
            if spec is not None:
                named[role] = (category, spec)
        self.arrangement = arrangement
        self.parts = named

    def __getattr__(self, role: str) -> PartSpec:
        parts = self.__dict__.get("parts", {})
        if role in parts:
            return parts[role][1]
        raise AttributeError(role)

    def roles(self, category: str) -> List[str]:
        return [role for role, (cat, _) in self.parts.items() if cat == category]


@dataclass(frozen=True)
class LayerRun:
    layer: int                        # index into ModelSpec.layers
    reads_cache_of: Optional[int] = None   # index of an earlier run whose cache this run reads instead of its own


@dataclass(frozen=True)
class ModelSpec:
    width: int
    vocab_size: int
    embedding: PartSpec
    position: PartSpec
    layers: Tuple[LayerSpec, ...]
    order: Tuple[LayerRun, ...]
    final_norm: PartSpec
    head: PartSpec
    max_positions: Optional[int] = None
    # (duplicate name, tensor it must equal): names a checkpoint may carry beside the tensor they alias
    tied_aliases: Tuple[Tuple[str, str], ...] = ()


@dataclass(frozen=True)
class CacheGroupSpec:
    """Runs whose mixers keep the same kind of pages share a page table and a pool geometry."""
    n_kv_head: int
    head_dim: int
    window: int
    n_pools: int       # caches (one per writing run) in the group


@dataclass
class CacheLayout:
    groups: List[CacheGroupSpec]
    state_numels: List[int]                        # one entry per (run, mixer) that keeps per-request state
    run_bindings: List[Dict[str, CacheBinding]]    # per run: mixer role -> where it keeps what it remembers

    @property
    def bindings(self) -> List[CacheBinding]:
        """One binding per run, for models whose layers have exactly one mixer each."""
        return [next(iter(b.values())) if len(b) == 1 else None for b in self.run_bindings]


@dataclass(frozen=True)
class KVRun:
    """One mixer of one run that reads keys and values."""
    n_head: int
    n_kv_head: int
    head_dim: int
    window: int


@dataclass(frozen=True)
class ModelCost:
    """What a step of the model has to read and to compute, taken from its parts and its order (for
    measurements against the machine's peaks; a dense model: every token goes through every matrix)."""
    whole_tensor_bytes: int       # tensors that a step reads whole (matrices, gains, biases; a table only where a
                                  # part also multiplies by it, as a tied head does), each once
    table_row_bytes: int          # bytes a token reads from the tables that are looked up by row only
    run_matrix_elements: int      # matrix elements a token goes through in the layers, over all runs of the order
    head_matrix_elements: int     # matrix elements a wanted logit row goes through behind the last run
    kv_runs: Tuple[KVRun, ...]    # every (run, mixer) that reads keys and values, its own cache or another run's

    def step_read_bytes(self, n_tokens: int, context_lens, cache_itemsize: int) -> float:
        """Bytes that a step of n_tokens single tokens has to read when request i has context_lens[i]
        keys to look at (its own included): every whole tensor once, the tokens' table rows, and
        for every run that attends the keys and values in its reach."""
        kv = 0.0
        for run in self.kv_runs:
            for c in context_lens:
                reach = min(c, run.window) if run.window else c
                kv += reach * 2 * run.n_kv_head * run.head_dim * cache_itemsize
        return self.whole_tensor_bytes + n_tokens * self.table_row_bytes + kv

    def prompt_flops(self, prompt_lens, n_logit_rows: int) -> float:
        """Multiply-adds times two of whole prompts in one step: the matrices for every token, causal
        attention (scores and weighted values for the keys a query sees), the head for the wanted rows."""
        n = sum(prompt_lens)
        flops = 2.0 * n * self.run_matrix_elements + 2.0 * n_logit_rows * self.head_matrix_elements
        for run in self.kv_runs:
            for t in prompt_lens:
                seen = sum(min(i + 1, run.window) if run.window else i + 1 for i in range(t))
                flops += 4.0 * seen * run.n_head * run.head_dim
        return flops


class _Layer:
    """The built parts of a layer, by role (also as attributes)."""

    def __init__(self, arrangement: Part, parts: Dict[str, Part]) -> None:
        self.arrangement = arrangement
        self.parts = parts

    def __getattr__(self, role: str) -> Part:
        parts = self.__dict__.get("parts", {})
        if role in parts:
            return parts[role]
        raise AttributeError(role)


class DecoderModel:
    def __init__(self, spec: ModelSpec) -> None:
        self.spec = spec
        self.embedding = EMBEDDINGS.build(spec.embedding)
        self.position = POSITIONS.build(spec.position)
        self.layers: List[_Layer] = []
        for i, ls in enumerate(spec.layers):
            arrangement = ARRANGEMENTS.build(ls.arrangement)
            wanted = getattr(arrangement, "roles", None)
            if wanted is not None and set(wanted) != set(ls.parts):
                raise ValueError(f"layer {i}: arrangement {ls.arrangement.kind!r} arranges the parts "
                                 f"{sorted(wanted)}, the layer has {sorted(ls.parts)}")
            self.layers.append(_Layer(arrangement, {role: _LAYER_REGISTRIES[category].build(part_spec)
                                                    for role, (category, part_spec) in ls.parts.items()}))
        self.final_norm = NORMS.build(spec.final_norm)
        self.head = HEADS.build(spec.head)
        for i, run in enumerate(spec.order):
            if not (0 <= run.layer < len(self.layers)):
                raise ValueError(f"run {i} names layer {run.layer}, but there are {len(self.layers)} layers")
            if run.reads_cache_of is not None and not (0 <= run.reads_cache_of < i):
                raise ValueError(f"run {i} can only read the cache of an earlier run, not {run.reads_cache_of}")
        self.cache_layout = self._plan_cache()

    # ------------------------------------------------------------------ weights
    def _named_parts(self) -> List[Tuple[Part, PartSpec]]:
        pairs = [(self.embedding, self.spec.embedding), (self.position, self.spec.position)]
        for layer, ls in zip(self.layers, self.spec.layers):
            pairs += [(layer.parts[role], part_spec) for role, (_, part_spec) in ls.parts.items()]
        pairs += [(self.final_norm, self.spec.final_norm), (self.head, self.spec.head)]
        return pairs

    def weight_requests(self) -> Dict[str, WeightRequest]:
        """Checkpoint tensor name -> shape and role, over all parts.  Two parts may name the same
        tensor (a tied head); then shape and role must agree."""
        wanted: Dict[str, WeightRequest] = {}
        for part, spec in self._named_parts():
            for local, req in part.weight_requests().items():
                if local not in spec.weights:
                    raise KeyError(f"{spec.kind}: no checkpoint name given for parameter {local!r}")
                name = spec.weights[local]
                if name in wanted and (wanted[name].shape != req.shape):
                    raise ValueError(f"tensor {name} is asked for with shapes {wanted[name].shape} and {req.shape}")
                if name not in wanted or req.role == "table":
                    wanted[name] = req
        return wanted

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self._bound = {name: tensors[name] for name in self.weight_requests()}
        for part, spec in self._named_parts():
            part.bind({local: tensors[spec.weights[local]] for local in part.weight_requests()})

    def weight_bytes(self) -> Tuple[int, int]:
        """(bytes of the tensors as loaded, bytes of the copies derived from them since: matrices
        folded with a LayerNorm or packed for the decode kernels, made at first use).  A tensor that
        two parts share (a tied head) counts once."""
        from ..ops.linear import derived_bytes

        loaded = derived = 0
        seen = set()
        for tensor in getattr(self, "_bound", {}).values():
            if tensor.data_ptr() in seen:
                continue
            seen.add(tensor.data_ptr())
            loaded += tensor.numel() * tensor.element_size()
            derived += derived_bytes(tensor)
        return loaded, derived

    def cost(self) -> ModelCost:
        """The model's bytes and multiply-adds per step, from the bound tensors and the order of runs."""
        bound = getattr(self, "_bound", None)
        if bound is None:
            raise RuntimeError("cost() needs the model's tensors (bind)")
        whole, by_row = set(), set()
        for part, spec in self._named_parts():
            for local, req in part.weight_requests().items():
                (by_row if req.role == "table" else whole).add(spec.weights[local])
        by_row -= whole
        size = lambda name: bound[name].numel() * bound[name].element_size()
        row_bytes = sum(size(name) // bound[name].shape[0] for name in by_row)

        def matrices(part: Part) -> int:
            total = 0
            for req in part.weight_requests().values():
                if req.role == "matrix":
                    n = 1
                    for dim in req.shape:
                        n *= dim
                    total += n
            return total

        run_elements, kv_runs = 0, []
        for run in self.spec.order:
            layer = self.layers[run.layer]
            for part in layer.parts.values():
                run_elements += matrices(part)
                need = part.cache_need() if hasattr(part, "cache_need") else None
                if isinstance(need, KVNeed):
                    kv_runs.append(KVRun(int(getattr(part, "n_head", need.n_kv_head)), need.n_kv_head,
                                         need.head_dim, need.window))
        return ModelCost(sum(size(name) for name in whole), row_bytes, run_elements, matrices(self.head),
                         tuple(kv_runs))

    # ------------------------------------------------------------------ cache
    def _plan_cache(self) -> CacheLayout:
        groups: List[CacheGroupSpec] = []
        keys: List[Tuple[int, int, int]] = []
        state_numels: List[int] = []
        run_bindings: List[Dict[str, CacheBinding]] = []
        for i, run in enumerate(self.spec.order):
            layer, layer_spec = self.layers[run.layer], self.spec.layers[run.layer]
            bindings: Dict[str, CacheBinding] = {}
            for role in layer_spec.roles("mixer"):
                need = layer.parts[role].cache_need()
                if run.reads_cache_of is not None:
                    src_run = self.spec.order[run.reads_cache_of]
                    src = run_bindings[run.reads_cache_of].get(role)
                    src_need = (self.layers[src_run.layer].parts[role].cache_need()
                                if role in self.layers[src_run.layer].parts else None)
                    if src is None or need != src_need or src.kind != "kv":
                        raise ValueError(f"run {i} cannot read the cache of run {run.reads_cache_of}: different needs")
                    bindings[role] = CacheBinding("kv", src.group, src.index, writes=False)
                elif isinstance(need, KVNeed):
                    key = (need.n_kv_head, need.head_dim, need.window)
                    if key not in keys:
                        keys.append(key)
                        groups.append(CacheGroupSpec(need.n_kv_head, need.head_dim, need.window, 0))
                    g = keys.index(key)
                    bindings[role] = CacheBinding("kv", g, groups[g].n_pools, writes=True)
                    groups[g] = CacheGroupSpec(*key, groups[g].n_pools + 1)
                elif isinstance(need, StateNeed):
                    bindings[role] = CacheBinding("state", -1, len(state_numels), writes=True)
                    state_numels.append(int(need.numel))
                else:
                    bindings[role] = CacheBinding("none")
            run_bindings.append(bindings)
        return CacheLayout(groups, state_numels, run_bindings)

    @property
    def graph_safe(self) -> bool:
        """Whether every part of the model allows a step to be captured in a HIP graph (Part.graph_safe)."""
        parts = [self.embedding, self.position, self.final_norm, self.head]
        for layer in self.layers:
            parts += [layer.arrangement, *layer.parts.values()]
        return all(getattr(p, "graph_safe", False) for p in parts if p is not None)

    @property
    def plan_safe(self) -> bool:
        """Whether every part of the model computes through the kernel library only (Part.plan_safe)."""
        parts = [self.embedding, self.position, self.final_norm, self.head]
        for layer in self.layers:
            parts += [layer.arrangement, *layer.parts.values()]
        return self.graph_safe and all(getattr(p, "plan_safe", False) for p in parts if p is not None)

    # ------------------------------------------------------------------ forward
    def forward(self, ctx: StepContext) -> torch.Tensor:
        """Runs the step's tokens through every run of the order and returns float32 logits
        [m_rows, vocab] at ctx.logit_rows (reference: src/minigpt_infer/model.py:183-187, there for
        the last position only)."""
        n = ctx.n_rows
        ws = ctx.workspace
        x = ws.get("residual", n, self.spec.width, torch.float32)
        ctx.pending = None
        self.embedding.forward(ctx, self.position, x)
        for run, bindings in zip(self.spec.order, self.cache_layout.run_bindings):
            layer = self.layers[run.layer]
            if not layer.arrangement.takes_pending_residual:
                residual.settle(ctx, x, n)
            layer.arrangement.run(ctx, x, layer.parts, bindings, self.position)
        m = ctx.m_rows
        # rows start 16 bytes apart at least: the sampling kernel then reads them four floats at a time
        # whatever the vocabulary's size (50257 is odd)
        vocab = self.spec.vocab_size
        logits = ws.get("logits", m, -(-vocab // 4) * 4, torch.float32)[:, :vocab]
        if m:
            # every token's logits wanted, in order (the host has looked at the list): row i of the
            # logits is token i, and the norm need not wait for the list before it can send for its rows
            rows = None if ctx.decode_only and m == n and ctx.logit_rows_in_order else ctx.logit_rows
            self.head.forward(ctx, LazyNorm(self.final_norm, x, m, rows=rows, buffer="final_normed"), logits, m)
        ctx.pending = None
        return logits[:m]

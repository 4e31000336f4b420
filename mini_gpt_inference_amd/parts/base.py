"""What a model is put together from: part specifications, the registries that
turn a specification into a part, and the step context every part receives.

A part knows its own sizes and constants (they are constructor parameters) and
the names of its weights inside itself; it does not know which model it is in,
which layer it is, or what the other parts are.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Callable, Dict, List, Optional, Tuple

import torch

# roles of a weight tensor: how the loader stores it on the device
MATRIX = "matrix"   # compute dtype (bfloat16 when serving, float32 on the 32-bit path)
VECTOR = "vector"   # always float32: gains, biases
TABLE = "table"     # compute dtype, looked up by row


@dataclass(frozen=True)
class PartSpec:
    """kind: registry key; params: sizes and constants; weights: parameter name -> checkpoint tensor name."""
    kind: str
    params: Dict[str, Any] = field(default_factory=dict)
    weights: Dict[str, str] = field(default_factory=dict)


@dataclass(frozen=True)
class WeightRequest:
    shape: Tuple[int, ...]
    role: str


@dataclass(frozen=True)
class KVNeed:
    """A mixer that keeps keys and values of past tokens in pages."""
    n_kv_head: int
    head_dim: int
    window: int = 0   # 0: all earlier keys; w: the last w positions


@dataclass(frozen=True)
class StateNeed:
    """A mixer that keeps a fixed number of float32 values per request."""
    numel: int


class Part:
    """Base of every part.  Subclasses set `category` and implement their forward."""

    category = "part"
    # True if forward() launches the same kernels with the same arguments for every step of the same
    # shape (the numbers of tokens each request brings and of logit rows), taking all else (positions,
    # lengths, slots, tables) from the step's device arrays: then a step may be captured in a HIP
    # graph and replayed.  A part that looks at ctx.host_ctx_lens or ctx.host_state_slots, or that
    # allocates, is not.
    graph_safe = False
    # True if, beyond graph_safe, forward() computes through the kernel library's launchers only
    # (ops.kernels), with no operator of the tensor library: then a step's launches can be recorded
    # once and made again from C++ (ops.plan.LaunchPlan), which sees no other work than theirs.
    plan_safe = False
    # True if the part reads the residual stream through ops.residual (it takes sums that are still
    # pending, or settles them itself); every other part is handed a plain residual stream
    takes_pending_residual = False

    def weight_requests(self) -> Dict[str, WeightRequest]:
        """Parameter name -> shape and role of every tensor this part needs."""
        return {}

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        """Receives the device tensors named by weight_requests (absent optional ones are missing)."""
        for name, tensor in tensors.items():
            setattr(self, name, tensor)


class Registry:
    def __init__(self, category: str) -> None:
        self.category = category
        self._kinds: Dict[str, Callable[..., Part]] = {}

    def register(self, kind: str) -> Callable:
        def deco(cls):
            if kind in self._kinds and self._kinds[kind] is not cls:
                raise ValueError(f"{self.category} kind {kind!r} is already registered")
            self._kinds[kind] = cls
            return cls
        return deco

    def build(self, spec: PartSpec) -> Part:
        if spec.kind not in self._kinds:
            raise KeyError(f"no {self.category} of kind {spec.kind!r}; known: {sorted(self._kinds)}")
        return self._kinds[spec.kind](**spec.params)

    def kinds(self) -> List[str]:
        return sorted(self._kinds)


NORMS = Registry("norm")
MIXERS = Registry("mixer")
FEED_FORWARDS = Registry("feed-forward")
POSITIONS = Registry("position encoding")
ARRANGEMENTS = Registry("block arrangement")
EMBEDDINGS = Registry("embedding")
HEADS = Registry("output head")

register_norm = NORMS.register
register_mixer = MIXERS.register
register_feed_forward = FEED_FORWARDS.register
register_position = POSITIONS.register
register_arrangement = ARRANGEMENTS.register
register_embedding = EMBEDDINGS.register
register_head = HEADS.register


@dataclass
class GroupView:
    """One cache group as a step sees it."""
    page_size: int
    window: int
    slot_mapping: torch.Tensor   # [n_stride] int32: flat slot of each token, -1 = padding
    block_tables: torch.Tensor   # [r_stride, max_blocks] int32, -1 = no page
    k_pools: List[torch.Tensor]  # per cache slot of the group: [pages, kv_heads, page_size, head_dim]
    v_pools: List[torch.Tensor]


@dataclass
class CacheBinding:
    """Where one run of a layer keeps what its mixer remembers."""
    kind: str            # "kv", "state" or "none"
    group: int = -1      # cache group (kv)
    index: int = -1      # pool index inside the group (kv) or state pool index (state)
    writes: bool = True  # False: the run reads a cache that an earlier run of this step wrote


class WorkspaceFrozen(RuntimeError):
    """A buffer would have to be (re)allocated while a HIP graph holds the workspace's addresses."""


class Workspace:
    """Named scratch buffers that grow on demand and are reused from step to step."""

    def __init__(self, device: torch.device) -> None:
        self.device = device
        self._buffers: Dict[tuple, torch.Tensor] = {}
        self.frozen = False   # set while a HIP graph owns the addresses
        self.generation = 0   # counts (re)allocations: a graph captured before one holds stale addresses

    def get(self, name: str, rows: int, cols: int, dtype: torch.dtype) -> torch.Tensor:
        # one buffer per (name, width, dtype): layers of different widths that use the same name
        # must not take each other's buffer away (a step graph holds the addresses of both)
        key = (name, cols, dtype)
        buf = self._buffers.get(key)
        if buf is None or buf.shape[0] < rows:
            if self.frozen:
                raise WorkspaceFrozen(f"workspace buffer {name!r} would have to grow while a graph holds it")
            buf = torch.empty((rows, cols), dtype=dtype, device=self.device)
            self._buffers[key] = buf
            self.generation += 1
        return buf


@dataclass
class StepContext:
    """Everything a part may read about the step it runs in.

    Token-indexed arrays have n_stride entries of which the first n_tokens are real;
    request-indexed ones r_stride / n_req; logit rows m_stride / n_logits."""
    n_tokens: int                # real tokens of the step
    n_rows: int                  # rows every part processes: n_tokens, or the padded count of a graph bucket
    n_req: int
    n_logits: int                # real logit rows
    m_rows: int                  # logit rows computed: n_logits, or the padded count
    token_ids: torch.Tensor      # [n_stride] int32
    positions: torch.Tensor      # [n_stride] int32, absolute position of each token
    q_req: torch.Tensor          # [n_stride] int32, index of the token's request in this step, -1 = padding
    cu_q: torch.Tensor           # [r_stride + 1] int32, token offsets of the requests
    seq_lens: torch.Tensor       # [r_stride] int32, length of each request after this step
    state_slots: torch.Tensor    # [r_stride] int32, the request's slot in every state pool
    logit_rows: torch.Tensor     # [m_stride] int32, tokens whose logits are wanted
    groups: List[GroupView]
    state_pools: List[torch.Tensor]   # per state binding: [max_requests, numel] float32
    dtype: torch.dtype           # compute dtype of activations and matrices
    workspace: Workspace
    max_q_len: int               # host-side bounds used to size launches
    max_seq_len: int
    decode_only: bool            # every request brings exactly one token
    # host copies for parts written with library calls (tests' toy parts)
    host_q_lens: Optional[List[int]] = None
    host_ctx_lens: Optional[List[int]] = None
    host_state_slots: Optional[List[int]] = None
    exact: bool = False          # true 32-bit path: no fast-math intrinsics
    padded: bool = False         # rows and requests are padded to a bucket's sizes (n_rows, cu_q.numel() - 1):
                                 # the host values above then describe the bucket, not the step
    lead_cap: int = 0            # padded steps: the decoding requests' tokens lie among the first lead_cap
    # sums that are still to be added to the residual stream (ops.residual.PendingSums); None: it is plain
    pending: Optional[Any] = None
    # the host has seen that logit_rows is 0, 1, ..., n_tokens - 1 (every token's logits, in order)
    logit_rows_in_order: bool = False
    # an ops.linear.CopyBudget: device memory that copies of matrices made at first use may still take;
    # None: no bound
    copy_budget: Optional[Any] = None
    # set by a caller that will choose greedily among the logits: an ops.linear.TileBest, which the
    # head fills beside the logits if its kernel can
    tile_best: Optional[Any] = None

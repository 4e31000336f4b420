"""Engine tuning knobs and per-request sampling options.

Names and meanings follow the reference: ``EngineConfig`` (block_size,
num_blocks, max_batch_size; src/minigpt_infer/config.py:21-29) and
``SamplingParams`` (src/minigpt_infer/config.py:32-41).  The token budget, the
prefill portion size and the mixed-batch switch have no counterpart there: the
reference never cuts a prompt and never mixes prompt work with decoding
(src/minigpt_infer/engine/scheduler.py:9-12).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Optional


@dataclass
class EngineConfig:
    block_size: int = 16             # tokens per KV page (the reference's "KV block")
    num_blocks: int = 2048           # pages in the fixed pool, per cache group (the reference's num_blocks)
    kv_cache_bytes: Optional[int] = None   # instead of num_blocks: device memory for all cache groups together,
                                           # split so that every group holds the same number of full-length
                                           # requests (groups differ in bytes per token and in their window)
    max_batch_size: int = 256        # most requests running at once (= state slots)
    max_num_batched_tokens: int = 4096   # token budget of one step
    prefill_chunk: int = 0           # largest prompt portion per request and step; 0 = no limit
    mixed_batches: bool = True       # False: a step with admissions runs prompts only,
                                     # as the reference does (scheduler.py:52-56)
    evict: str = "newest"            # when pages run out during decoding: "newest" evicts the newest running
                                     # request, also when it is the one that asks; "newest_other" never the
                                     # asker while another runs, as the reference does (scheduler.py:66-82)
    dtype: str = "bfloat16"          # "bfloat16" (serving) or "float32" (true 32-bit path)
    use_graph: bool = True           # replay decode-only steps, and other steps whose shape repeats, from
                                     # captured HIP graphs
    decode_burst: int = 8            # decode steps captured as one graph and enqueued back to back when
                                     # nothing else is pending, tokens fed on the device from one to the
                                     # next; 1 = off
    decode_chain: int = 4            # such graphs enqueued one behind the other before the host waits: it
                                     # launches the next and takes in the tokens of the last while the
                                     # device is at work
    decode_ahead: bool = True        # before the host waits for a chain's last tokens it plans and enqueues
                                     # the next chain, whose tokens the next step() call returns
    derived_weight_bytes: Optional[int] = None   # most device memory for the copies of matrices that the decode
                                     # kernels make at first use (packed for their loads, folded with a
                                     # LayerNorm: up to 1.5 times the weights); None = no bound, 0 = no copies:
                                     # the decode steps then read the matrices as loaded, more slowly
    seed: int = 0                    # engine-wide sampler seed
    real_vocab_size: Optional[int] = None  # ids at or above it are never sampled
                                           # (src/minigpt_infer/tokenizer.py:37-46)

    def __post_init__(self) -> None:
        if self.block_size <= 0 or self.num_blocks <= 0 or self.max_batch_size <= 0:
            raise ValueError("block_size, num_blocks and max_batch_size must be positive")
        if self.kv_cache_bytes is not None and self.kv_cache_bytes <= 0:
            raise ValueError("kv_cache_bytes must be positive")
        if self.max_num_batched_tokens <= 0:
            raise ValueError("max_num_batched_tokens must be positive")
        if self.decode_burst < 1 or self.decode_chain < 1:
            raise ValueError("decode_burst and decode_chain must be at least 1")
        if self.derived_weight_bytes is not None and self.derived_weight_bytes < 0:
            raise ValueError("derived_weight_bytes must be >= 0")
        if self.prefill_chunk < 0:
            raise ValueError("prefill_chunk must be >= 0")
        if self.evict not in ("newest", "newest_other"):
            raise ValueError(f"evict must be 'newest' or 'newest_other', got {self.evict!r}")
        if self.dtype in ("bf16",):
            self.dtype = "bfloat16"
        if self.dtype in ("fp32",):
            self.dtype = "float32"
        if self.dtype not in ("bfloat16", "float32"):
            raise ValueError(f"dtype must be bfloat16 or float32, got {self.dtype!r}")


@dataclass
class SamplingParams:
    max_tokens: int = 128
    temperature: float = 1.0         # 0.0 => greedy (src/minigpt_infer/sampling.py:120)
    top_k: Optional[int] = None
    top_p: Optional[float] = None
    seed: Optional[int] = None       # per-request sampler stream; None = derived from the request's arrival order
    n: int = 1

    def __post_init__(self) -> None:
        if self.n != 1:
            # src/minigpt_infer/engine/engine.py:70
            raise ValueError("n>1 completions per request are not supported")
        if self.max_tokens <= 0:
            raise ValueError("max_tokens must be positive")
        if self.top_k is not None and self.top_k <= 0:
            raise ValueError("top_k must be positive")
        if self.top_p is not None and not (0.0 < self.top_p <= 1.0):
            raise ValueError("top_p must lie in (0, 1]")

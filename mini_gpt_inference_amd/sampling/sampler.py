"""Next-token choice on the device (csrc/hip/sampling.hip): greedy where temperature <= 0,
otherwise temperature, top-k, top-p and a seeded draw."""

from __future__ import annotations

import torch

from ..ops import kernels


class Sampler:
    def __init__(self, vocab_size: int, real_vocab_size=None, engine_seed: int = 0) -> None:
        self.vocab_size = vocab_size
        self.real_vocab = vocab_size if real_vocab_size is None else int(real_vocab_size)
        if not (0 < self.real_vocab <= vocab_size):
            raise ValueError("real_vocab_size must lie in 1..vocab_size")
        self.engine_seed = int(engine_seed)

    def sample(self, logits: torch.Tensor, arena, n_rows: int, advance=None, tile_best=None) -> torch.Tensor:
        """Writes one token per logits row into arena.tokens_out, using the arena's per-row sampling
        arrays.  Returns arena.tokens_out.  advance = (page_sizes, history): after a decode-only
        step, also turn the arena's device arrays into those of the next step and append the
        tokens to history [steps, rows] (see kernels.sample).  tile_best: an ops.linear.TileBest that
        the head has filled for these logits with this sampler's real_vocab as its limit."""
        d = arena.d
        adv = None
        if advance is not None:
            page_sizes, history = advance
            adv = (d["token_ids"], d["positions"], d["seq_lens"], d["q_req"],
                   d["slot_mapping"].view(arena.n_groups, arena.n_cap),
                   d["block_tables"].view(arena.n_groups, arena.r_cap, arena.max_blocks), page_sizes, history,
                   d["history_pos"])
        kernels.sample(logits, n_rows, self.real_vocab, d["temperature"], d["top_k"], d["top_p"], d["seeds"],
                       d["out_index"], self.engine_seed, arena.tokens_out, advance=adv,
                       tile_best=(tile_best.values, tile_best.columns)
                       if tile_best is not None and tile_best.filled and tile_best.limit == self.real_vocab else None)
        return arena.tokens_out

"""LLMEngine: scheduler + cache + step function + sampler behind the reference's entry points
(add_request / step / has_unfinished_requests / cancel_request,
src/minigpt_infer/engine/engine.py:42-118), plus generate() and constructors from a model folder
or from a configuration and a seed.
"""

from __future__ import annotations

import contextlib
import shutil
import tempfile
import time
from typing import Dict, List, Optional, Sequence, Union

import numpy as np
import torch

from ..cache.kv_store import KVStore
from ..cache.manager import CacheManager, GroupGeometry, plan_group_pages
from ..config.engine_config import EngineConfig, SamplingParams
from ..ops import kernels, library
from ..ops.linear import TileBest
from ..ops.plan import LaunchPlan
from ..parts.base import Workspace
from ..sampling.sampler import Sampler
from ..weights.loader import load_model
from ..weights.random_init import write_random_model
from .request import Request, RequestOutput
from .scheduler import FINISHED, Scheduler
from .step import ModelRunner, StepArena, StepShape, _bucket

_TORCH_DTYPES = {"bfloat16": torch.bfloat16, "float32": torch.float32}


class _GraphedDecode:
    """Captured HIP graphs of a decode-only step (model + sampling) for up to `cap` requests.  The
    arena and the workspace are its own, so their addresses never change.  The sampling kernel also
    turns the arena's device arrays into the next step's (its token, position, length, cache slot)
    and appends the tokens to `history`, so that steps can follow each other with no copy between
    them: `burst` of them are captured as one graph as well."""

    def __init__(self, runner: ModelRunner, sampler: Sampler, cap: int, burst: int, chain: int = 1) -> None:
        self.runner, self.sampler, self.cap, self.burst = runner, sampler, cap, max(burst, 1)
        self.max_steps = self.burst * max(chain, 1)      # most steps enqueued from one upload
        self.arena = StepArena(cap, cap, cap, runner.n_groups, runner.max_blocks, runner.device)
        self.workspace = Workspace(runner.device)
        # two halves: a chain that goes on from the last one writes the other half, while the host
        # still reads that one's tokens
        self.history = torch.zeros(2 * self.max_steps, cap, dtype=torch.int32, device=runner.device)
        self.history_host = torch.zeros(2 * self.max_steps, cap, dtype=torch.int32,
                                        pin_memory=runner.device.type == "cuda")
        self.history_base = 0
        self.graph: Optional[torch.cuda.CUDAGraph] = None
        self.burst_graph: Optional[torch.cuda.CUDAGraph] = None
        self.shape: Optional[StepShape] = None   # of the last single step; launch geometry for captures
        self.kernels_per_step = 0                # kernels that the captured step launches
        self.plan: Optional[LaunchPlan] = None   # the step's launches, recorded at its one eager run
        self.tile_best_used = False              # greedy rows choose from what the head left per tile

    def _launch(self, shape: StepShape, record: bool = False) -> None:
        """The step's kernels (model and sampling) through the model's Python.  record: keep the
        launches as a plan, from which the captures make them again without the Python."""
        ctx = self.runner.context(self.arena, shape, padded=True, workspace=self.workspace)
        # launch geometry must not depend on this step's lengths: size it for the longest sequence
        ctx.max_seq_len = self.runner.max_positions or ctx.max_seq_len
        ctx.tile_best = TileBest(self.sampler.real_vocab)
        launched = kernels.launches
        with kernels.pinned_stream(), (library.record() if record else contextlib.nullcontext()) as launches:
            logits = self.runner.model.forward(ctx)
            self.sampler.sample(logits, self.arena, self.cap, advance=(self.runner.page_sizes, self.history),
                                tile_best=ctx.tile_best)
        self.kernels_per_step = kernels.launches - launched
        if record:
            self.plan = LaunchPlan(launches)
        self.tile_best_used = ctx.tile_best.filled

    def _capture(self, shape: StepShape, times: int) -> torch.cuda.CUDAGraph:
        self.runner.num_graph_captures += 1
        graph = torch.cuda.CUDAGraph()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            graph.capture_begin()
            try:
                for _ in range(times):
                    if self.plan is not None:
                        with kernels.pinned_stream():
                            self.plan.run()
                    else:
                        self._launch(shape)
            except BaseException:
                # never leave the stream capturing: the graph object's destructor synchronizes the
                # device, which a stream that is still capturing turns into an abort of the process
                try:
                    graph.capture_end()
                except RuntimeError:
                    pass
                raise
            graph.capture_end()
        torch.cuda.current_stream().wait_stream(side)
        return graph

    def run(self, shape: StepShape) -> None:
        """One step from the uploaded arena."""
        self.arena.h["history_pos"][:] = 0
        self.history_base = 0
        self.arena.upload()
        if self.graph is None:
            # once eagerly, so that every workspace buffer and every derived copy of a matrix exists
            # before capture; then once more, counted and recorded: the step as every later one runs
            self._launch(shape)
            torch.cuda.synchronize()
            self.workspace.frozen = True
            self.arena.upload()
            self._launch(shape, record=self.runner.plan_steps)
            torch.cuda.synchronize()
            self.graph = self._capture(shape, 1)
            # the eager launch above did this step's work and moved the device arrays on to the
            # next step: upload this step's again
            self.arena.upload()
        self.shape = shape
        self.graph.replay()

    def run_burst(self, k: int, ahead: bool = False):
        """k steps, each feeding the next on the device.  They are enqueued in stretches (whole
        captured bursts, then single steps); behind each stretch its rows of the history are copied
        to the host and an event is recorded.  Returns [(first row, end row, event)]: once a
        stretch's event has passed, history_host[first:end] holds its tokens, while the device is at
        work on the stretches behind it.  ahead: the steps go on from where the steps enqueued before
        them will end (their tokens, positions and cache slots are the device's own); only the block
        tables are uploaded, and the tokens go to the history's other half."""
        if self.graph is None:
            raise RuntimeError("a burst needs the single step's graph, which the first decode step captures")
        if k > self.max_steps:
            raise ValueError(f"{k} steps asked for, the history holds {self.max_steps}")
        base = (self.max_steps - self.history_base) if ahead else 0
        self.history_base = base
        self.arena.h["history_pos"][:] = base
        if ahead:
            self.arena.upload_tables()
        else:
            self.arena.upload()
        stretches, done = [], 0
        while done < k:
            if k - done >= self.burst > 1:
                if self.burst_graph is None:
                    self.burst_graph = self._capture(self.shape, self.burst)
                self.burst_graph.replay()
                end = done + self.burst
            else:
                end = done
                while end < k:      # the rest: single steps one behind the other, one copy and one event
                    self.graph.replay()
                    end += 1
            self.history_host[base + done:base + end].copy_(self.history[base + done:base + end], non_blocking=True)
            event = torch.cuda.Event()
            event.record()
            stretches.append((base + done, base + end, event))
            done = end
        return stretches


class LLMEngine:
    def __init__(self, model, config, engine_config: EngineConfig, device: str = "cuda") -> None:
        self.model, self.config, self.engine_config = model, config, engine_config
        self.device = torch.device(device)
        self.dtype = _TORCH_DTYPES[engine_config.dtype]
        layout = model.cache_layout
        pages = plan_group_pages(layout.groups, engine_config.block_size, engine_config.num_blocks,
                                 engine_config.kv_cache_bytes, 2 if self.dtype == torch.bfloat16 else 4,
                                 model.spec.max_positions)
        geometry = [GroupGeometry(engine_config.block_size, n, g.window) for g, n in zip(layout.groups, pages)]
        self.cache = CacheManager(geometry, engine_config.max_batch_size)
        self.store = KVStore(layout, geometry, engine_config.max_batch_size, self.dtype, self.device)
        max_positions = model.spec.max_positions
        self.runner = ModelRunner(model, self.cache, self.store, self.dtype, self.device, max_positions,
                                  graph_steps=engine_config.use_graph,
                                  derived_weight_bytes=engine_config.derived_weight_bytes)
        self.scheduler = Scheduler(
            self.cache, engine_config.max_batch_size,
            max(engine_config.max_num_batched_tokens, engine_config.max_batch_size),
            engine_config.prefill_chunk, engine_config.mixed_batches,
            max_positions if max_positions is not None else 2 ** 30,
            spare_asker=engine_config.evict == "newest_other")
        self.sampler = Sampler(model.spec.vocab_size, engine_config.real_vocab_size, engine_config.seed)
        self._ids: Dict[int, str] = {}        # scheduler id -> caller's request id
        self._rids: Dict[str, int] = {}
        self._generated = 0                   # requests that generate() has named so far
        self._inflight = None                 # a chain of decode steps enqueued ahead, not yet taken in
        self._graphs: Dict[int, _GraphedDecode] = {}
        self._unseeded = 0                    # requests so far that brought no seed of their own
        self._tmpdir: Optional[str] = None
        self.num_graph_steps = 0
        self.num_eager_steps = 0
        # a list here collects (decode steps, time.perf_counter()) whenever the tokens of a stretch of
        # enqueued decode steps have arrived on the host: the device's pace, for measurements
        self.stretch_times: Optional[List] = None

    # ------------------------------------------------------------------ constructors
    @classmethod
    def from_folder(cls, model_dir: str, engine_config: Optional[EngineConfig] = None,
                    device: str = "cuda") -> "LLMEngine":
        engine_config = engine_config or EngineConfig()
        model, config, _ = load_model(model_dir, engine_config.dtype, device)
        return cls(model, config, engine_config, device)

    @classmethod
    def from_random(cls, config, seed: int, engine_config: Optional[EngineConfig] = None,
                    device: str = "cuda", std_scale: float = 1.0) -> "LLMEngine":
        """Random weights: writes a model folder from (config, seed), then loads it like any other."""
        tmp = tempfile.mkdtemp(prefix="mgpt_random_")
        try:
            write_random_model(tmp, config, seed, std_scale=std_scale)
            return cls.from_folder(tmp, engine_config, device)
        finally:
            shutil.rmtree(tmp, ignore_errors=True)

    # ------------------------------------------------------------------ requests
    def add_request(self, request: Request) -> None:
        if request.request_id in self._rids:
            raise ValueError(f"request id {request.request_id!r} is already in use")
        sp = request.sampling_params
        vocab = self.model.spec.vocab_size
        if any((t < 0 or t >= vocab) for t in request.prompt_token_ids):
            raise ValueError(f"prompt token id outside 0..{vocab - 1}")
        seed = sp.seed
        if seed is None:
            # a stream of its own per request in the order of arrival; the made-up requests of
            # capture_decode_graphs bring a seed, so that calling it changes nobody's tokens
            seed = self._unseeded
            self._unseeded += 1
        sid = self.scheduler.add_request(request.prompt_token_ids, sp.max_tokens, request.eot_token_id,
                                         sp.temperature, sp.top_k, sp.top_p, seed)
        self._ids[sid] = request.request_id
        self._rids[request.request_id] = sid

    def has_unfinished_requests(self) -> bool:
        return self.scheduler.has_work()

    def cancel_request(self, request_id: str) -> bool:
        sid = self._rids.get(request_id)
        return False if sid is None else self.scheduler.cancel(sid)

    # ------------------------------------------------------------------ stepping
    def _launch_chain(self, max_steps: Optional[int], ahead: bool):
        """Plans up to decode_burst x decode_chain decode steps (at most max_steps) and enqueues them.
        ahead: behind a chain whose last tokens the host has not seen yet.  Returns (graphs, requests,
        steps, stretches), or None when no burst can be planned now."""
        ecfg = self.engine_config
        if ecfg.decode_burst < 2 or not ecfg.use_graph or not self._graphs:
            return None
        r = len(self.scheduler.running)
        graphed = self._graphs.get(_bucket(max(r, 1)))
        if graphed is None or graphed.graph is None:
            return None
        k = self.scheduler.plan_burst(graphed.max_steps if max_steps is None else min(graphed.max_steps, max_steps))
        if k < 2:
            return None
        self.scheduler.fill(graphed.arena)
        self.num_graph_steps += k
        return graphed, r, k, graphed.run_burst(k, ahead=ahead)

    def _try_burst(self, max_steps: Optional[int] = None) -> Optional[List[RequestOutput]]:
        """Several decode steps enqueued at once: one upload, the captured steps (each prepares the
        next one's inputs on the device); their tokens come back stretch by stretch and are handed to
        the scheduler while the device runs the stretches behind.  Before the host waits for the last
        stretch it plans and enqueues the next chain (decode_ahead), which the next call then takes
        in: as long as nothing else comes up, the device never waits for the host.  max_steps: the
        most steps this call may plan; 0 only takes in what is enqueued."""
        chain, self._inflight = self._inflight, None
        if chain is None:
            if max_steps is not None and max_steps < 2:
                return None
            chain = self._launch_chain(max_steps, ahead=False)
            if chain is None:
                return None
            if max_steps is not None:
                max_steps -= chain[2]
        graphed, r, k, stretches = chain
        outs: List[RequestOutput] = []
        for i, (first, end, event) in enumerate(stretches):
            last = i == len(stretches) - 1
            if last and self.engine_config.decode_ahead and (max_steps is None or max_steps >= 2):
                self._inflight = self._launch_chain(max_steps, ahead=True)
            event.synchronize()
            if self.stretch_times is not None:
                self.stretch_times.append((end - first, time.perf_counter()))
            tokens = np.ascontiguousarray(graphed.history_host.numpy()[first:end, :r])
            outs += [RequestOutput(self._ids[sid], [token], finished, reason) for sid, token, finished, reason
                     in self.scheduler.commit_burst(tokens, end - first, last=last)]
        # a chain enqueued ahead for requests that have all ended since brings nothing: the caller goes on
        # with an ordinary step
        return outs if outs or self._inflight is not None else None

    def step(self, max_decode_steps: Optional[int] = None) -> List[RequestOutput]:
        """One step of the engine: admits, runs one batch (or, when every running request is decoding
        and nobody waits, up to decode_burst x decode_chain decode steps back to back), hands the
        sampled tokens to the scheduler.  Returns one RequestOutput per token sampled.  With
        decode_ahead a call may also enqueue the decode steps whose tokens the next call returns.
        max_decode_steps bounds the decode steps that this call newly plans, those enqueued ahead
        included; 0 only takes in what an earlier call enqueued."""
        burst = self._try_burst(max_decode_steps)
        if burst is not None or max_decode_steps == 0:
            return burst or []
        n, r, m = self.scheduler.schedule()
        if r == 0:
            return []
        decode_only = n == r
        use_graph = decode_only and self.engine_config.use_graph and m == r and self.model.graph_safe
        if use_graph:
            cap = _bucket(r)
            graphed = self._graphs.get(cap)
            if graphed is None:
                graphed = self._graphs[cap] = _GraphedDecode(self.runner, self.sampler, cap,
                                                             self.engine_config.decode_burst,
                                                             self.engine_config.decode_chain)
            arena = graphed.arena
        else:
            arena = self.runner.arena(n, r, m)
        self.scheduler.fill(arena)
        _, ctx_lens, q_lens, _ = self.scheduler.entry_arrays()
        slots = arena.h["state_slots"][:r]
        shape = self.runner.shape_of(arena, n, r, m, q_lens.tolist(), ctx_lens.tolist(), slots.tolist())
        if use_graph:
            graphed.run(shape)
            self.num_graph_steps += 1
        else:
            logits = self.runner.run(arena, shape)
            if m:
                self.sampler.sample(logits, arena, m)
            self.num_eager_steps += 1
        if m:
            arena.tokens_host.copy_(arena.tokens_out, non_blocking=True)
        torch.cuda.current_stream().synchronize()
        tokens = arena.tokens_host.numpy()[:m]
        outs = []
        for sid, token, finished, reason in self.scheduler.commit(tokens):
            rid = self._ids[sid]
            outs.append(RequestOutput(rid, [token], finished, reason))
        return outs

    def generate(self, prompts: Sequence[Sequence[int]],
                 sampling_params: Union[SamplingParams, Sequence[SamplingParams], None] = None,
                 eot_token_id: Optional[int] = None) -> List[List[int]]:
        """Runs the prompts to completion and returns the new token ids of each, in order."""
        if sampling_params is None:
            sampling_params = SamplingParams()
        params = (list(sampling_params) if isinstance(sampling_params, (list, tuple))
                  else [sampling_params] * len(prompts))
        if len(params) != len(prompts):
            raise ValueError("one SamplingParams per prompt, or one for all")
        names = [f"generate-{self._generated + i}" for i in range(len(prompts))]
        self._generated += len(prompts)
        got: Dict[str, List[int]] = {name: [] for name in names}
        for name, prompt, sp in zip(names, prompts, params):
            self.add_request(Request(name, list(prompt), sp, eot_token_id))
        while self.has_unfinished_requests():
            outs = self.step()
            for out in outs:
                if out.request_id in got:
                    got[out.request_id].extend(out.new_token_ids)
            if not outs and not self.scheduler.running:
                raise RuntimeError("the scheduler cannot make progress: the waiting request does not fit")
        self.forget_finished()
        return [got[name] for name in names]

    def capture_decode_graphs(self, batch_sizes: Optional[Sequence[int]] = None) -> List[int]:
        """Captures the graphs of decode steps ahead of time, as a server does before it takes
        requests (the reference's CUDAGraphRunner.capture does it for one batch size,
        src/minigpt_infer/graphs.py:96-110): for every capacity that decode steps are padded to (the
        powers of two up to max_batch_size, or those that hold the given batch sizes) it runs that many
        made-up one-token requests for a few steps, which captures the single step and the burst.
        A capacity whose requests the page pool cannot hold is left out.  Returns the capacities
        captured.  The engine must be idle; its counters count these steps too.  The tokens of later
        requests do not depend on whether this was called."""
        ecfg = self.engine_config
        if self.has_unfinished_requests() or self._inflight is not None:
            raise RuntimeError("capture_decode_graphs needs an idle engine")
        if not ecfg.use_graph or not self.model.graph_safe:
            return []
        if batch_sizes is None:
            caps, c = [], 1
            while c < ecfg.max_batch_size:
                caps.append(c)
                c *= 2
            caps.append(c)
        else:
            caps = sorted({_bucket(max(int(b), 1)) for b in batch_sizes})
        steps = max(ecfg.decode_burst, 1) * max(ecfg.decode_chain, 1) + 3
        if self.runner.max_positions is not None:
            steps = min(steps, self.runner.max_positions - 1)
        done: List[int] = []
        for cap in caps:
            n = min(cap, ecfg.max_batch_size)
            if steps < 2 or _bucket(n) != cap:
                continue
            if any(n * self.cache.pages_needed(1 + steps, g) > self.cache.num_free_pages(g)
                   for g in range(len(self.cache.groups))):
                continue
            for i in range(n):
                self.add_request(Request(f"capture-{cap}-{i}-{self._generated}", [0],
                                         SamplingParams(max_tokens=steps, temperature=0.0, seed=0)))
            self._generated += 1
            while self.has_unfinished_requests():
                self.step()
            self.forget_finished()
            if cap in self._graphs and self._graphs[cap].graph is not None:
                done.append(cap)
        return done

    def forget_finished(self) -> int:
        """Drops what the engine still holds of finished requests (their ids and token lists), so that
        an engine that serves for a long time does not grow; their ids may be used again.  Returns
        how many were dropped.  generate() calls it; a loop around step() calls it when it likes."""
        done = [sid for sid in self._ids if self.scheduler.info(sid).status == FINISHED]
        for sid in done:
            del self._rids[self._ids.pop(sid)]
        self.scheduler.forget_finished()
        return len(done)

    # ------------------------------------------------------------------ counters
    def fragmentation_stats(self, group: int = 0) -> Dict[str, int]:
        """Free and allocated pages of a cache group and the slots that allocated pages hold beyond the
        tokens computed into them (src/minigpt_infer/cache/paged.py:83-94)."""
        geometry = self.cache.groups[group]
        free = self.cache.num_free_pages(group)
        allocated = geometry.num_pages - free
        computed = 0
        for sid in self.scheduler.running:
            n = self.scheduler.info(sid).num_computed
            computed += min(n, geometry.window) if geometry.window else n
        return {"free_blocks": free, "allocated_blocks": allocated,
                "internal_fragmentation_slots": max(0, allocated * geometry.page_size - computed)}

    def stats(self) -> Dict[str, int]:
        s = self.scheduler
        weight_bytes, derived_bytes = self.model.weight_bytes()
        return {
            # device memory of the weights as loaded, and of the copies made of them at first use
            # (packed for the decode kernels, folded with a LayerNorm)
            "weight_bytes": weight_bytes, "derived_weight_bytes": derived_bytes,
            "cache_bytes": self.store.bytes(),
            "num_preemptions": s.num_preemptions, "num_steps": s.num_steps,
            "num_prompt_tokens": s.num_prompt_tokens, "num_decode_tokens": s.num_decode_tokens,
            "free_blocks": self.cache.num_free_pages(0),
            "allocated_blocks": self.cache.groups[0].num_pages - self.cache.num_free_pages(0),
            "graph_steps": self.num_graph_steps, "eager_steps": self.num_eager_steps,
            "replayed_eager_steps": self.runner.num_replayed_steps,
            "graph_captures": self.runner.num_graph_captures,
        }

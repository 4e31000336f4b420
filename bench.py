"""Decode and prefill throughput of the engine on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one decode step of the engine (scheduler, one step of the model from the cache,
sampling, tokens back on the host).  The default run has the layer sizes of the reference's
50.9M model (n_layer 8, n_embd 512, n_head 8, vocabulary 50304, 1024 positions, biases) with
random weights in bfloat16, a batch of 8 requests with 128-token random prompts, KV pages of 16
tokens.  It prints one JSON line; `value` is decoded tokens per second.  Beside it: the
prefill of 2,048 tokens (2 prompts of 1,024) as one step, the decode step's bytes against the
HBM peak, and decode throughput at batch 1 and 64.

    python bench.py --workload small-mixed | xl-preempt

runs one of the family's other two named workloads end to end (see WORKLOADS) and prints its own line.
"""

from __future__ import annotations

import argparse
import json
import sys
import time

HBM_PEAK_GBS = 8000.0                      # MI355X HBM3E
MFMA_PEAK = {"bfloat16": 2.5e15, "float32": 157.3e12}   # dense, per second
REFERENCE_DECODE_B8 = 1671.8               # tok/s, the reference's own figure (Tesla T4, fp16, batch 8)


def build_engine(args, batch, dtype):
    from mini_gpt_inference_amd import EngineConfig, GPTConfig
    from mini_gpt_inference_amd.engine.llm_engine import LLMEngine

    cfg = GPTConfig("gpt2-mini", n_layer=args.layers, n_embd=args.width, n_head=args.heads,
                    vocab_size=args.vocab, block_size=args.positions, bias=True, layer_norm_eps=1e-5)
    pages = batch * (-(-args.positions // args.kv_block)) + 8
    ecfg = EngineConfig(block_size=args.kv_block, num_blocks=pages, max_batch_size=max(batch, 2),
                        max_num_batched_tokens=max(4096, batch * args.prompt), dtype=dtype,
                        use_graph=not args.no_graph, decode_burst=args.burst, decode_chain=args.chain)
    return LLMEngine.from_random(cfg, seed=0, engine_config=ecfg), cfg


def decode_run(args, batch, steps, warmup, dtype):
    """Returns (seconds for `steps` decode steps, mean context length during them, engine, cfg)."""
    import numpy as np
    import torch

    from mini_gpt_inference_amd import Request, SamplingParams

    engine, cfg = build_engine(args, batch, dtype)
    if not args.no_graph:
        # every graph that the timed steps replay (the single step's and the burst's) is recorded
        # here, before any request: the reference captures before it times as well
        # (src/minigpt_infer/graphs.py:96-110)
        assert engine.capture_decode_graphs([batch]), "the decode graphs could not be captured ahead"
    rng = np.random.default_rng(0)
    budget = steps + warmup + 3 * args.burst * args.chain + 2
    assert args.prompt + budget <= cfg.block_size, "prompt + decode steps exceed the model's positions"
    for i in range(batch):
        engine.add_request(Request(f"b{i}", rng.integers(0, cfg.vocab_size, args.prompt).tolist(),
                                   SamplingParams(max_tokens=budget, temperature=0.0)))
    sched = engine.scheduler
    decoded_before = sched.num_decode_tokens
    while sched.num_decode_tokens == decoded_before:      # prompts, untimed
        engine.step()

    samples = []     # (decode steps in the call, seconds) of every engine.step() call of the timed region

    def run_decode_steps(n, record=False):
        """engine.step() until exactly n more decode steps have run (a call may run a burst of them)."""
        first, tokens = sched.num_steps, sched.num_decode_tokens
        while sched.num_steps - first < n:
            before, t_call = sched.num_steps, time.perf_counter()
            engine.step(max_decode_steps=n - (sched.num_steps - first))
            if record:
                samples.append((sched.num_steps - before, time.perf_counter() - t_call))
        engine.step(max_decode_steps=0)      # what the last call enqueued ahead is taken in here
        assert sched.num_steps - first == n, "the decode bursts do not divide the number of steps"
        assert sched.num_decode_tokens - tokens == n * batch, "a request dropped out of the decode steps"

    done = sched.num_steps
    run_decode_steps(warmup)
    torch.cuda.synchronize()
    start_ctx = args.prompt + 1 + (sched.num_steps - done)
    before = engine.stats()
    engine.stretch_times = stretches = []
    t0 = time.perf_counter()
    run_decode_steps(steps, record=True)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    engine.stretch_times = None
    after = engine.stats()
    assert after["graph_captures"] == before["graph_captures"], "a HIP graph was recorded inside the timed steps"
    if not args.no_graph:
        assert after["graph_steps"] - before["graph_steps"] == steps, "a timed step did not come from a graph"
    engine.step_samples = samples
    # the device's pace: from the arrival of one stretch's tokens (a captured burst, or the single
    # steps that end a chain) to the arrival of the next one's
    engine.stretch_samples = [(n, t1 - t_prev) for (_, t_prev), (n, t1) in zip(stretches, stretches[1:])]
    mean_ctx = start_ctx + (steps - 1) / 2.0 + 1     # keys read per request and step, own token included
    return elapsed, mean_ctx, engine, cfg


def kernels_per_step(engine, batch):
    """Kernels that one captured decode step of this batch launches (0 without graphs)."""
    from mini_gpt_inference_amd.engine.step import _bucket

    graphed = engine._graphs.get(_bucket(max(batch, 1)))
    return graphed.kernels_per_step if graphed is not None else 0


def decode_bytes(cfg, batch, mean_ctx, itemsize):
    """Bytes one decode step has to read: every weight it uses once (the position table is not
    among them), and the keys and values of the live requests."""
    c, f, L = cfg.n_embd, 4 * cfg.n_embd, cfg.n_layer
    per_layer = (3 * c * c + c * c + 2 * f * c) * itemsize + (3 * c + c + f + c + 4 * c) * 4
    weights = L * per_layer + cfg.vocab_size * c * itemsize + 2 * c * 4
    kv = batch * mean_ctx * 2 * L * c * itemsize
    return weights + kv


def prefill_run(args, dtype, reps=9):
    import numpy as np
    import torch

    n_req = args.prefill_requests
    engine, cfg = build_engine(args, n_req, dtype)
    runner, cache = engine.runner, engine.cache
    t_len = min(1024, cfg.block_size)
    rng = np.random.default_rng(1)
    tokens = rng.integers(0, cfg.vocab_size, n_req * t_len).astype(np.int32)   # prompts held as arrays, not lists
    times = []
    for rep in range(reps + 2):
        slots = [cache.acquire_slot() for _ in range(n_req)]
        for s in slots:
            assert cache.reserve(s, t_len)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        runner.step(slots, [0] * n_req, [t_len] * n_req, tokens, [(i + 1) * t_len - 1 for i in range(n_req)])
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
        for s in slots:
            cache.free_slot(s)
    best = sorted(times[2:])[len(times[2:]) // 2]
    n = n_req * t_len
    c, L = cfg.n_embd, cfg.n_layer
    flops = n * 24 * c * c * L + n_req * (2 * t_len * t_len * c) * L + n_req * 2 * c * cfg.vocab_size
    return {"value": round(n / best, 1), "tokens": n, "ms": round(best * 1e3, 4),
            "frac": round(flops / best / MFMA_PEAK[dtype], 5)}


WORKLOADS = {
    # the reference family's other two named workloads (shapes of GPT-2 small and GPT-2 XL, random weights)
    "small-mixed": dict(layers=12, width=768, heads=12, vocab=50257, positions=1024, requests=64,
                        prompt=(16, 1024), output=(16, 256), prefill_chunk=512, pool_frac=1.0),
    "xl-preempt": dict(layers=48, width=1600, heads=25, vocab=50257, positions=1024, requests=256,
                       prompt=(512, 512), output=(512, 512), prefill_chunk=0, pool_frac=0.55),
}


def serve_run(args, name):
    """A whole continuous-batching run: all requests arrive at once, prompts are cut into portions
    beside the decoding of others, requests end at their own lengths; with pool_frac < 1 the page
    pool is smaller than the requests' full demand, so the newest are evicted and recomputed."""
    import numpy as np
    import torch

    from mini_gpt_inference_amd import EngineConfig, GPTConfig, Request, SamplingParams
    from mini_gpt_inference_amd.engine.llm_engine import LLMEngine

    w = dict(WORKLOADS[name])
    if args.workload_layers:
        w["layers"] = args.workload_layers
    if args.workload_requests:
        w["requests"] = args.workload_requests
    cfg = GPTConfig("gpt2-mini", n_layer=w["layers"], n_embd=w["width"], n_head=w["heads"], vocab_size=w["vocab"],
                    block_size=w["positions"], bias=True, layer_norm_eps=1e-5)
    rng = np.random.default_rng(2)
    requests = []
    for i in range(w["requests"]):
        p = int(rng.integers(w["prompt"][0], w["prompt"][1] + 1))
        o = int(rng.integers(w["output"][0], w["output"][1] + 1))
        p = min(p, cfg.block_size - o)          # prompt + output within the model's positions
        requests.append((rng.integers(0, cfg.vocab_size, p).tolist(), o))
    demand = sum(-(-(len(p) + o) // args.kv_block) for p, o in requests)
    pages = max(int(demand * w["pool_frac"]), -(-cfg.block_size // args.kv_block) + 1)
    ecfg = EngineConfig(block_size=args.kv_block, num_blocks=pages, max_batch_size=w["requests"],
                        max_num_batched_tokens=4096, prefill_chunk=w["prefill_chunk"], dtype=args.dtype,
                        use_graph=not args.no_graph, decode_burst=args.burst, decode_chain=args.chain)
    engine = LLMEngine.from_random(cfg, seed=0, engine_config=ecfg)
    if not args.no_capture:
        engine.capture_decode_graphs()      # before the clock starts, as a server does before it takes requests
    before = engine.stats()
    for i, (p, o) in enumerate(requests):
        engine.add_request(Request(f"r{i}", p, SamplingParams(max_tokens=o, temperature=0.0)))
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    produced = 0
    while engine.has_unfinished_requests():
        produced += len(engine.step())
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    stats = {key: value - before[key] if key.startswith(("num_", "graph_", "eager_", "replayed_")) else value
             for key, value in engine.stats().items()}
    assert produced == sum(o for _, o in requests), "a request ended early or late"
    assert stats["free_blocks"] == pages, "pages were lost"
    return {"workload": name, "value": round(produced / elapsed, 1), "unit": "generated tokens/s",
            "seconds": round(elapsed, 3), "requests": len(requests), "generated_tokens": produced,
            "prompt_tokens": sum(len(p) for p, _ in requests), "n_layer": cfg.n_layer, "n_embd": cfg.n_embd,
            "n_head": cfg.n_head, "vocab_size": cfg.vocab_size, "pages": pages, "page_demand": demand,
            "steps": stats["num_steps"], "decode_graph_steps": stats["graph_steps"],
            "other_steps_replayed": stats["replayed_eager_steps"], "preemptions": stats["num_preemptions"],
            "prompt_tokens_computed": stats["num_prompt_tokens"], "dtype": args.dtype, "weights": "random"}


def host_cost_run(args):
    """What the host pays to launch one mixed step of the GPT-2-small shape (eight single tokens
    beside a prompt portion of 300, no HIP graph): through the model's Python, and from the plan
    recorded at the shape's first coming (one call into the kernel library).  Host time is the time
    until the launching call returns; the device is idle before each."""
    import numpy as np
    import torch

    from mini_gpt_inference_amd import EngineConfig, GPTConfig
    from mini_gpt_inference_amd.engine.llm_engine import LLMEngine
    from mini_gpt_inference_amd.ops import kernels

    w = WORKLOADS["small-mixed"]
    layers = args.workload_layers or w["layers"]
    cfg = GPTConfig("gpt2-mini", n_layer=layers, n_embd=w["width"], n_head=w["heads"], vocab_size=w["vocab"],
                    block_size=w["positions"], bias=True, layer_norm_eps=1e-5)
    engine = LLMEngine.from_random(cfg, seed=0, engine_config=EngineConfig(
        block_size=args.kv_block, num_blocks=1024, max_batch_size=16, dtype=args.dtype, use_graph=False))
    runner, cache = engine.runner, engine.cache
    rng = np.random.default_rng(3)
    q_lens = [1] * 8 + [300]
    ctx_lens = [int(c) for c in rng.integers(20, 200, 8)] + [212]
    slots = [cache.acquire_slot() for _ in q_lens]
    for s, c, q in zip(slots, ctx_lens, q_lens):
        assert cache.reserve(s, c + q)
    tokens = rng.integers(0, cfg.vocab_size, sum(q_lens)).astype(np.int32)
    rows = list(range(8)) + [sum(q_lens) - 1]

    def one(plans):
        runner.plan_steps = plans
        torch.cuda.synchronize()
        before, t0 = kernels.launches, time.perf_counter()
        runner.step(slots, ctx_lens, q_lens, tokens, rows)
        host = time.perf_counter() - t0
        torch.cuda.synchronize()
        return host, kernels.launches - before, time.perf_counter() - t0

    one(True)                                   # first coming: buffers made, matrices packed, the plan recorded
    one(True)
    python_runs = [one(False) for _ in range(args.host_cost_reps)]
    planned_before = runner.num_planned_steps
    plan_runs = [one(True) for _ in range(args.host_cost_reps)]
    assert runner.num_planned_steps - planned_before == args.host_cost_reps, "the steps did not come from the plan"
    med = lambda runs, i: sorted(r[i] for r in runs)[len(runs) // 2]
    n_kernels = plan_runs[0][1]      # launcher calls (one whose product is split along k is two kernels)
    # the launches alone, without describing the step and uploading its arrays
    plan = runner._entry((tuple(q_lens), len(rows))).plan
    alone = []
    for _ in range(args.host_cost_reps):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        plan.run()
        alone.append(time.perf_counter() - t0)
    torch.cuda.synchronize()
    alone_us = sorted(alone)[len(alone) // 2] * 1e6
    return {"workload": "host cost of an eager mixed step", "n_layer": cfg.n_layer, "n_embd": cfg.n_embd,
            "tokens": int(sum(q_lens)), "requests": len(q_lens), "kernels": n_kernels, "dtype": args.dtype,
            "python_host_us": round(med(python_runs, 0) * 1e6, 1),
            "python_host_us_per_kernel": round(med(python_runs, 0) * 1e6 / n_kernels, 2),
            "plan_host_us": round(med(plan_runs, 0) * 1e6, 1),
            "plan_host_us_per_kernel": round(med(plan_runs, 0) * 1e6 / n_kernels, 2),
            "plan_launches_alone_us": round(alone_us, 1), "plan_launches_alone_us_per_kernel": round(alone_us / n_kernels, 2),
            "python_step_us": round(med(python_runs, 2) * 1e6, 1), "plan_step_us": round(med(plan_runs, 2) * 1e6, 1)}


def main() -> int:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--layers", type=int, default=8)
    ap.add_argument("--width", type=int, default=512)
    ap.add_argument("--heads", type=int, default=8)
    ap.add_argument("--vocab", type=int, default=50304)
    ap.add_argument("--positions", type=int, default=1024)
    ap.add_argument("--prompt", type=int, default=128)
    ap.add_argument("--kv-block", type=int, default=16)
    ap.add_argument("--no-graph", action="store_true")
    ap.add_argument("--burst", type=int, default=8, help="decode steps captured as one graph (1 = off)")
    ap.add_argument("--chain", type=int, default=4, help="such graphs enqueued before the host waits")
    ap.add_argument("--no-extras", action="store_true", help="skip prefill and the batch 1 / 64 points")
    ap.add_argument("--workload", choices=sorted(WORKLOADS), default=None,
                    help="instead of the decode measurement: a whole continuous-batching run with the shape "
                         "of GPT-2 small (64 mixed requests, prompt portions of 512) or of GPT-2 XL (256 "
                         "requests, a page pool too small for them: evictions)")
    ap.add_argument("--no-capture", action="store_true",
                    help="--workload: leave the decode graphs to be captured inside the timed run")
    ap.add_argument("--workload-layers", type=int, default=0, help="fewer layers for --workload (0 = the shape's)")
    ap.add_argument("--workload-requests", type=int, default=0, help="fewer requests for --workload")
    ap.add_argument("--host-step-cost", action="store_true",
                    help="instead of the decode measurement: the host's time to launch an eager mixed step of the "
                         "GPT-2-small shape, through the model's Python and from its recorded plan")
    ap.add_argument("--host-cost-reps", type=int, default=15)
    ap.add_argument("--report", default=None,
                    help="also write a JSON file with the raw timing samples, their median and quartiles, the "
                         "commit and the software and device that ran them")
    ap.add_argument("--prefill-requests", type=int, default=2,
                    help="prompts of 1,024 tokens in the prefill step (the contract's 2,048 tokens are 2)")
    ap.add_argument("--prefill-only", action="store_true",
                    help="run only the 2,048-token prefill and print its record (for profiling)")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2

    if args.prefill_only:
        print(json.dumps({"prefill": prefill_run(args, args.dtype, reps=10)}))
        return 0
    if args.host_step_cost:
        print(json.dumps(host_cost_run(args)))
        return 0
    if args.workload:
        print(json.dumps(serve_run(args, args.workload)))
        return 0

    elapsed, mean_ctx, engine, cfg = decode_run(args, args.batch, args.steps, args.warmup, args.dtype)
    samples = engine.stretch_samples or engine.step_samples
    itemsize = 2 if args.dtype == "bfloat16" else 4
    step_s = elapsed / args.steps
    value = args.batch * args.steps / elapsed
    achieved = decode_bytes(cfg, args.batch, mean_ctx, itemsize) / step_s / 1e9
    stats = engine.stats()
    record = {
        "metric": f"decode tokens/s (50.9M GPT-2-style, batch {args.batch}, {args.prompt}-token prompts)",
        "value": round(value, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(step_s * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": round(value / REFERENCE_DECODE_B8, 2) if args.batch == 8 else None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic",
        "config": {
            "model": "gpt2-mini-50.9M", "n_layer": cfg.n_layer, "n_layer_full": 8, "n_embd": cfg.n_embd,
            "n_head": cfg.n_head, "head_dim": cfg.head_dim, "mlp_hidden": 4 * cfg.n_embd,
            "vocab_size": cfg.vocab_size, "block_size": cfg.block_size, "bias": True,
            "global_batch": args.batch, "seq_len": cfg.block_size, "prompt_len": args.prompt,
            "mean_context": round(mean_ctx, 1), "kv_block": args.kv_block, "weights": "random",
            "hip_graph": bool(stats["graph_steps"]), "decode_burst": args.burst, "decode_chain": args.chain,
            "parallelism": "single-gpu",
        },
        "kernels_per_step": kernels_per_step(engine, args.batch),
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 5)},
    }
    del engine
    if not args.no_extras:
        record["prefill"] = prefill_run(args, args.dtype)
        points = {}
        for b in (1, 64):
            k = min(args.steps, 128)
            el, _, eng, _ = decode_run(args, b, k, min(args.warmup, 8), args.dtype)
            points[f"decode_b{b}"] = round(b * k / el, 1)
            del eng
        record["points"] = points
    print(json.dumps(record))
    if args.report:
        write_report(args.report, record, samples)
    return 0


def write_report(path, record, samples):
    """The record, the raw samples behind it (one per stretch of decode steps enqueued at once, a
    captured burst mostly: decode steps, seconds from the arrival of the stretch before it on the
    host to its own), their median and quartiles per step, and what ran them (the reference's timing
    rules: warm-up, synchronisation around the timed region, median and quartiles over at least 30
    repeats, docs/PLAN.md:720-732, bench/common.py:118-157)."""
    import statistics
    import subprocess

    import torch

    per_step = sorted(sec / n for n, sec in samples if n)
    quart = statistics.quantiles(per_step, n=4) if len(per_step) >= 2 else [per_step[0]] * 3
    import os

    sha = os.environ.get("MGPT_GIT_SHA", "")      # where the tree is a copy without its history
    if not sha:
        try:
            sha = subprocess.run(["git", "rev-parse", "HEAD"], capture_output=True, text=True, timeout=10,
                                 cwd=os.path.dirname(os.path.abspath(__file__))).stdout.strip()
        except Exception:
            sha = ""
    # what identifies the code where there is no history: the digest of the native sources and flags
    # that the loaded kernel library was built from
    from mini_gpt_inference_amd.csrc import build
    try:
        with open(build.KERNEL_LIB + ".digest", encoding="ascii") as fh:
            kernels_digest = fh.read().strip()
    except OSError:
        kernels_digest = ""
    report = {"record": record,
              "ms_per_step": {"median": quart[1] * 1e3, "q1": quart[0] * 1e3, "q3": quart[2] * 1e3,
                              "calls": len(per_step)},
              "samples": [[n, sec] for n, sec in samples],
              "environment": {"git": sha, "kernel_sources_sha256": kernels_digest, "torch": torch.__version__, "hip": torch.version.hip,
                              "device": torch.cuda.get_device_name(0)}}
    with open(path, "w", encoding="utf-8") as fh:
        json.dump(report, fh, indent=1)


if __name__ == "__main__":
    sys.exit(main())

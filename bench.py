"""Decode and prefill throughput of the engine on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one decode step of the engine (scheduler, one step of the model from the cache,
sampling, tokens back on the host).  The default run has the layer sizes of the reference's
50.9M model (n_layer 8, n_embd 512, n_head 8, vocabulary 50304, 1024 positions, biases) with
random weights in bfloat16, a batch of 8 requests with 128-token random prompts, KV pages of 16
tokens, every request generating 256 tokens.  After W untimed decode steps the rest of a
generation is timed in blocks of exactly K steps, each bracketed by a synchronisation, and new
requests follow until 30 blocks are timed; `value` is decoded tokens per second of the median
block, `iqr_ms` the distance of the blocks' quartiles per step (the reference's timing rule,
bench/common.py:118-157).  It prints one JSON line.  Beside the decode figure: the prefill of
2,048 tokens (2 prompts of 1,024) as one step, the decode step's bytes against the HBM peak, and
decode throughput at batch 1 and 64.  Bytes and multiply-adds come from the model itself
(DecoderModel.cost), so --model-config measures any registered architecture the same way.

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


def raw_model_config(args, **override):
    """The config.json dict of the model to measure: the file --model-config names (any registered
    architecture), or the reference's 50.9M model with the sizes of the command line."""
    if args.model_config:
        with open(args.model_config, encoding="utf-8") as fh:
            raw = json.load(fh)
    else:
        raw = {"architecture": "gpt2-mini", "n_layer": args.layers, "n_embd": args.width, "n_head": args.heads,
               "vocab_size": args.vocab, "block_size": args.positions, "bias": True, "layer_norm_eps": 1e-5}
    raw.update(override)
    return raw


def build_engine(args, batch, dtype, raw=None, **engine_options):
    """(engine, typed config, architecture) with random weights; everything below the config.json dict
    goes through the registry, as for a model folder."""
    from mini_gpt_inference_amd import EngineConfig
    from mini_gpt_inference_amd.config.registry import architecture_of
    from mini_gpt_inference_amd.engine.llm_engine import LLMEngine

    raw = raw or raw_model_config(args)
    arch = architecture_of(raw)
    cfg = arch.config_from_json(raw)
    positions = arch.model_spec(cfg).max_positions or args.positions
    options = dict(block_size=args.kv_block, num_blocks=batch * (-(-positions // args.kv_block)) + 8,
                   max_batch_size=max(batch, 2), max_num_batched_tokens=max(4096, batch * args.prompt), dtype=dtype,
                   use_graph=not args.no_graph, decode_burst=args.burst, decode_chain=args.chain,
                   derived_weight_bytes=args.derived_weight_bytes)
    options.update(engine_options)
    return LLMEngine.from_random(cfg, seed=0, engine_config=EngineConfig(**options)), cfg, arch


def quartiles(values):
    """(first quartile, median, third quartile)."""
    import statistics

    if len(values) < 2:
        return values[0], values[0], values[0]
    q1, med, q3 = statistics.quantiles(values, n=4)
    return q1, med, q3


def decode_run(args, batch, steps, warmup, dtype, min_blocks):
    """Decode throughput by the reference's timing rule (warm-up, then the median and the quartiles
    over at least 30 timed repeats, each bracketed by synchronisation, the prompts' prefill outside
    the clock: bench/common.py:118-157, bench/bench_hardware.py:96-128): `batch` requests with
    --prompt random tokens generate --generate tokens each (128 and 256 by default); after `warmup`
    untimed decode steps the remaining ones are timed in blocks of exactly `steps`; new requests follow
    until min_blocks blocks are timed.  Returns a dict: the seconds of every block, the mean context
    length over the timed steps, the engine, its config and architecture."""
    import numpy as np
    import torch

    from mini_gpt_inference_amd import Request, SamplingParams

    engine, cfg, arch = build_engine(args, batch, dtype)
    spec = engine.model.spec
    if not args.no_graph:
        # every graph that the timed steps replay (the single step's and the burst's) is recorded
        # here, before any request: the reference captures before it times as well
        # (src/minigpt_infer/graphs.py:96-110)
        assert engine.capture_decode_graphs([batch]), "the decode graphs could not be captured ahead"
    generate = max(args.generate, warmup + steps + 1)      # the first token comes from the prompt's step
    assert spec.max_positions is None or args.prompt + generate <= spec.max_positions, \
        "prompt + generated tokens exceed the model's positions"
    rng = np.random.default_rng(0)
    sched = engine.scheduler
    blocks, contexts, stretches_all = [], [], []

    def run_decode_steps(n):
        """engine.step() until exactly n more decode steps have run (a call may run a burst of them)."""
        first, tokens = sched.num_steps, sched.num_decode_tokens
        while sched.num_steps - first < n:
            engine.step(max_decode_steps=n - (sched.num_steps - first))
        engine.step(max_decode_steps=0)      # what the last call enqueued ahead is taken in here
        assert sched.num_steps - first == n, "the decode bursts do not divide the number of steps"
        assert sched.num_decode_tokens - tokens == n * batch, "a request dropped out of the decode steps"

    round_no = 0
    while len(blocks) < min_blocks:
        for i in range(batch):
            engine.add_request(Request(f"r{round_no}-{i}", rng.integers(0, spec.vocab_size, args.prompt).tolist(),
                                       SamplingParams(max_tokens=generate, temperature=0.0)))
        decoded_before = sched.num_decode_tokens
        while sched.num_decode_tokens == decoded_before:      # prompts, untimed; their step samples the first token
            engine.step(max_decode_steps=1)
        done = (sched.num_decode_tokens - decoded_before) // batch      # decode steps of this generation so far
        if done < warmup:
            run_decode_steps(warmup - done)
            done = warmup
        per_round = (generate - 1 - done) // steps
        assert per_round >= 1
        torch.cuda.synchronize()
        before = engine.stats()
        for _ in range(per_round):
            engine.stretch_times = stretches = []
            t0 = time.perf_counter()
            run_decode_steps(steps)
            torch.cuda.synchronize()
            blocks.append(time.perf_counter() - t0)
            engine.stretch_times = None
            # keys a request reads in each of the block's steps, its own token included
            first = args.prompt + 1 + done
            contexts.append(first + (steps - 1) / 2.0)
            done += steps
            stretches_all += [(n, t1 - t_prev) for (_, t_prev), (n, t1) in zip(stretches, stretches[1:])]
        after = engine.stats()
        assert after["graph_captures"] == before["graph_captures"], "a HIP graph was recorded inside the timed steps"
        if not args.no_graph:
            assert after["graph_steps"] - before["graph_steps"] == per_round * steps, \
                "a timed step did not come from a graph"
        while engine.has_unfinished_requests():               # the rest of the generation, untimed
            engine.step()
        engine.forget_finished()
        round_no += 1
    return {"blocks": blocks, "mean_context": sum(contexts) / len(contexts), "engine": engine, "cfg": cfg,
            "arch": arch, "stretches": stretches_all, "generate": generate}


def kernels_per_step(engine, batch):
    """Kernels that one captured decode step of this batch launches (0 without graphs)."""
    from mini_gpt_inference_amd.engine.step import _bucket

    graphed = engine._graphs.get(_bucket(max(batch, 1)))
    return graphed.kernels_per_step if graphed is not None else 0


def prefill_run(args, dtype, reps=30, warmups=10):
    """One step of --prefill-requests whole prompts of 1,024 tokens (fewer where the model has fewer
    positions), logits at each prompt's last token: the median over `reps` repeats after `warmups`."""
    import numpy as np
    import torch

    n_req = args.prefill_requests
    engine, cfg, arch = build_engine(args, n_req, dtype)
    runner, cache, spec = engine.runner, engine.cache, engine.model.spec
    t_len = min(1024, spec.max_positions or 1024)
    rng = np.random.default_rng(1)
    tokens = rng.integers(0, spec.vocab_size, n_req * t_len).astype(np.int32)   # prompts held as arrays, not lists
    times = []
    for rep in range(reps + warmups):
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
    q1, med, q3 = quartiles(sorted(times[warmups:]))
    n = n_req * t_len
    flops = engine.model.cost().prompt_flops([t_len] * n_req, n_req)
    return {"value": round(n / med, 1), "tokens": n, "ms": round(med * 1e3, 4),
            "frac": round(flops / med / MFMA_PEAK[dtype], 5), "iqr_ms": round((q3 - q1) * 1e3, 4), "repeats": reps}


WORKLOADS = {
    # the reference family's other two named workloads (shapes of GPT-2 small and GPT-2 XL, random weights)
    "small-mixed": dict(layers=12, width=768, heads=12, vocab=50257, positions=1024, requests=64,
                        prompt=(16, 1024), output=(16, 256), prefill_chunk=512, pool_frac=1.0),
    "xl-preempt": dict(layers=48, width=1600, heads=25, vocab=50257, positions=1024, requests=256,
                       prompt=(512, 512), output=(512, 512), prefill_chunk=0, pool_frac=0.55),
}


def workload_model_config(w):
    """The config.json dict of a named workload's model (shapes of the gpt2-mini architecture)."""
    return {"architecture": "gpt2-mini", "n_layer": w["layers"], "n_embd": w["width"], "n_head": w["heads"],
            "vocab_size": w["vocab"], "block_size": w["positions"], "bias": True, "layer_norm_eps": 1e-5}


def architecture_config(raw):
    from mini_gpt_inference_amd.config.registry import architecture_of

    return architecture_of(raw).config_from_json(raw)


def serve_run(args, name):
    """A whole continuous-batching run: all requests arrive at once, prompts are cut into portions
    beside the decoding of others, requests end at their own lengths; with pool_frac < 1 the page
    pool is smaller than the requests' full demand, so the newest are evicted and recomputed."""
    import numpy as np
    import torch

    from mini_gpt_inference_amd import Request, SamplingParams

    w = dict(WORKLOADS[name])
    if args.workload_layers:
        w["layers"] = args.workload_layers
    if args.workload_requests:
        w["requests"] = args.workload_requests
    raw = workload_model_config(w)
    cfg = architecture_config(raw)
    rng = np.random.default_rng(2)
    requests = []
    for i in range(w["requests"]):
        p = int(rng.integers(w["prompt"][0], w["prompt"][1] + 1))
        o = int(rng.integers(w["output"][0], w["output"][1] + 1))
        p = min(p, cfg.block_size - o)          # prompt + output within the model's positions
        requests.append((rng.integers(0, cfg.vocab_size, p).tolist(), o))
    demand = sum(-(-(len(p) + o) // args.kv_block) for p, o in requests)
    pages = max(int(demand * w["pool_frac"]), -(-cfg.block_size // args.kv_block) + 1)
    engine, _, _ = build_engine(args, w["requests"], args.dtype, raw, num_blocks=pages, max_batch_size=w["requests"],
                                max_num_batched_tokens=4096, prefill_chunk=w["prefill_chunk"])
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

    from mini_gpt_inference_amd.ops import kernels

    w = dict(WORKLOADS["small-mixed"])
    w["layers"] = args.workload_layers or w["layers"]
    raw = workload_model_config(w)
    engine, cfg, _ = build_engine(args, 16, args.dtype, raw, num_blocks=1024, max_batch_size=16, use_graph=False)
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
    plan = runner._entry((tuple(q_lens), len(rows), False)).plan
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


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=32, help="decode steps of one timed block")
    ap.add_argument("--warmup", type=int, default=16, help="untimed decode steps before a generation's blocks")
    ap.add_argument("--blocks", type=int, default=30, help="timed blocks at least (median and quartiles over them)")
    ap.add_argument("--generate", type=int, default=256,
                    help="tokens every request generates (more if warm-up and one block need more)")
    ap.add_argument("--model-config", default=None,
                    help="a config.json of any registered architecture to measure instead of the 50.9M model "
                         "(random weights; --layers, --width, --heads, --vocab, --positions are then unused)")
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
    ap.add_argument("--derived-weight-bytes", type=int, default=None,
                    help="bound for the copies of matrices that the decode kernels make at first use (0 = none)")
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
    args = ap.parse_args(argv)
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2

    if args.prefill_only:
        print(json.dumps({"prefill": prefill_run(args, args.dtype)}))
        return 0
    if args.host_step_cost:
        print(json.dumps(host_cost_run(args)))
        return 0
    if args.workload:
        print(json.dumps(serve_run(args, args.workload)))
        return 0

    run = decode_run(args, args.batch, args.steps, args.warmup, args.dtype, args.blocks)
    engine, cfg, arch = run["engine"], run["cfg"], run["arch"]
    itemsize = 2 if args.dtype == "bfloat16" else 4
    q1, med, q3 = quartiles(sorted(run["blocks"]))
    step_s = med / args.steps
    value = args.batch * args.steps / med
    mean_ctx = run["mean_context"]
    cost = engine.model.cost()
    achieved = cost.step_read_bytes(args.batch, [mean_ctx] * args.batch, itemsize) / step_s / 1e9
    stats = engine.stats()
    spec = engine.model.spec
    raw = dict(arch.config_to_json(cfg))
    default_model = not args.model_config
    # the reference's 50.9M model: its widths (fewer layers are named beside the full count)
    reference_sizes = default_model and (args.width, args.heads, args.vocab, args.positions) == (512, 8, 50304, 1024) \
        and args.layers <= 8
    config = {"model": "gpt2-mini-50.9M" if reference_sizes else
              "gpt2-mini-other-sizes" if default_model else str(raw.get("architecture"))}
    # every size the architecture's config.json names, then what its code fixes (taken from the parts)
    config.update({k: v for k, v in raw.items() if k != "architecture" and isinstance(v, (int, float, str, bool))})
    config.pop("layer_norm_eps", None)
    layer0 = spec.layers[0].parts
    for key, role, param in (("head_dim", "mixer", "head_dim"), ("mlp_hidden", "feed_forward", "hidden")):
        if role in layer0 and param in layer0[role][1].params:
            config[key] = layer0[role][1].params[param]
    if "n_layer" in config:
        config["n_layer_full"] = 8 if reference_sizes else config["n_layer"]
    config.update({"global_batch": args.batch, "seq_len": spec.max_positions, "prompt_len": args.prompt,
                   "generated": run["generate"], "mean_context": round(mean_ctx, 1), "kv_block": args.kv_block,
                   "weights": "random", "hip_graph": bool(stats["graph_steps"]), "decode_burst": args.burst,
                   "parallelism": "single-gpu"})
    name = ("50.9M GPT-2-style" if reference_sizes and args.layers == 8 else
            f"50.9M GPT-2-style, {args.layers} of 8 layers" if reference_sizes else
            f"GPT-2-style, {args.layers} layers of width {args.width}" if default_model else config["model"])
    record = {
        "metric": f"decode tokens/s ({name}, batch {args.batch}, {args.prompt}-token prompts, "
                  f"{run['generate']} generated tokens)",
        "value": round(value, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(step_s * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": round(value / REFERENCE_DECODE_B8, 2) if args.batch == 8 and reference_sizes and args.layers == 8
        else None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic",
        "config": config,
        # the timing rule: `value` is from the median block of `steps` decode steps; the quartiles' distance per step
        "blocks": len(run["blocks"]), "iqr_ms": round((q3 - q1) / args.steps * 1e3, 4), "decode_chain": args.chain,
        "kernels_per_step": kernels_per_step(engine, args.batch),
        "weight_bytes": stats["weight_bytes"], "derived_weight_bytes": stats["derived_weight_bytes"],
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 5)},
    }
    samples = [(args.steps, sec) for sec in run["blocks"]]
    stretches = run["stretches"]
    del engine, run
    if not args.no_extras:
        record["prefill"] = prefill_run(args, args.dtype)
        points = {}
        for b in (1, 64):
            r = decode_run(args, b, args.steps, args.warmup, args.dtype, args.blocks)
            points[f"decode_b{b}"] = round(b * args.steps / quartiles(sorted(r["blocks"]))[1], 1)
            del r
        record["points"] = points
    print(json.dumps(record))
    if args.report:
        write_report(args.report, record, samples, stretches)
    return 0


def write_report(path, record, samples, stretches):
    """The record, the raw samples behind it (decode steps, seconds of every timed block), the
    device's own pace inside the blocks (one sample per stretch of decode steps enqueued at once, a
    captured burst mostly: decode steps, seconds from the arrival of the stretch before it on the host
    to its own), the blocks' median and quartiles per step, and what ran them (the reference's timing
    rules: warm-up, synchronisation around the timed region, median and quartiles over at least 30
    repeats, docs/PLAN.md:720-732, bench/common.py:118-157)."""
    import subprocess

    import torch

    per_step = sorted(sec / n for n, sec in samples if n)
    quart = quartiles(per_step)
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
              "stretches": [[n, sec] for n, sec in stretches],
              "environment": {"git": sha, "kernel_sources_sha256": kernels_digest, "torch": torch.__version__, "hip": torch.version.hip,
                              "device": torch.cuda.get_device_name(0)}}
    with open(path, "w", encoding="utf-8") as fh:
        json.dump(report, fh, indent=1)


if __name__ == "__main__":
    sys.exit(main())

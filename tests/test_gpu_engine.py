"""Generation through the entry points: greedy tokens against the plain implementation, seeded
sampling, what happens when pages run out, graph replay against eager steps, the command line."""

import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import helpers
import plain_gpt as P
from mini_gpt_inference_amd import EngineConfig, Request, SamplingParams
from mini_gpt_inference_amd.engine.llm_engine import LLMEngine
from mini_gpt_inference_amd.engine.scheduler import SchedulerError

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _prompts(name, lengths, seed=0):
    rng = np.random.default_rng(seed)
    return [helpers.random_ids(rng, helpers.CONFIGS[name].vocab_size, n) for n in lengths]


def _plain_greedy(folder, prompts, n_new):
    cfg, w = P.read_model_folder(folder)
    return [P.plain_greedy_generate(w, cfg, p, n_new) for p in prompts]


def _assert_greedy_within_tolerance(folder, prompt, tokens, dtype):
    """Every token the engine chose is, for the plain implementation's logits on the engine's own
    prefix, the best one or within twice the logit tolerance of the best: what a greedy choice can
    be when each logit is only known to that tolerance."""
    cfg, w = P.read_model_folder(folder)
    ids = list(prompt)
    exact = 0
    for tok in tokens:
        logits = P.plain_forward(w, cfg, ids)[-1].numpy()
        margin = 2 * helpers.TOL[dtype] * max(1.0, np.abs(logits).max())
        assert logits[tok] >= logits.max() - margin, (len(ids), tok, int(np.argmax(logits)))
        exact += tok == int(np.argmax(logits))
        ids.append(tok)
    return exact


@pytest.mark.parametrize("use_graph", [True, False])
def test_greedy_generation_32bit_equals_plain_tokens(model_folders, use_graph):
    # The family's first tiny workload: three requests of 5/17/30 tokens, 12 greedy tokens, pages of 4
    prompts = _prompts("A", [5, 17, 30])
    want = _plain_greedy(model_folders["A"], prompts, 12)
    engine = LLMEngine.from_folder(model_folders["A"], EngineConfig(block_size=4, num_blocks=64, max_batch_size=4,
                                                                    dtype="float32", use_graph=use_graph))
    assert engine.generate(prompts, SamplingParams(max_tokens=12, temperature=0.0)) == want
    assert engine.cache.num_free_pages() == 64 and engine.cache.check() == 0      # nothing leaked
    assert (engine.stats()["graph_steps"] > 0) == use_graph


@pytest.mark.parametrize("name", ["A", "B"])
def test_greedy_generation_bfloat16_chooses_the_plain_argmax_up_to_rounding(model_folders, name):
    lengths = {"A": [5, 17, 30, 2], "B": [1, 9, 33, 64, 100]}[name]
    prompts = _prompts(name, lengths, seed=4)
    n_new = 16
    engine = LLMEngine.from_folder(model_folders[name], EngineConfig(block_size=8, num_blocks=128, max_batch_size=8,
                                                                     prefill_chunk=16, dtype="bfloat16"))
    got = engine.generate(prompts, SamplingParams(max_tokens=n_new, temperature=0.0))
    exact = 0
    for prompt, tokens in zip(prompts, got):
        assert len(tokens) == n_new
        exact += _assert_greedy_within_tolerance(model_folders[name], prompt, tokens, "bfloat16")
    assert exact >= 0.9 * n_new * len(prompts)      # and nearly always it is the argmax itself


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("n_req", [20, 40])
def test_many_requests_decode_from_padded_graphs(model_folders, dtype, n_req):
    """20 and 40 requests: decode steps replayed from the graphs of 32 and 64 rows (padded), in chained
    bursts; requests end at different lengths, so later steps fall into smaller graphs."""
    rng = np.random.default_rng(31)
    prompts = _prompts("B", [int(n) for n in rng.integers(1, 40, n_req)], seed=32)
    news = [int(n) for n in rng.integers(3, 20, n_req)]
    engine = LLMEngine.from_folder(model_folders["B"], EngineConfig(block_size=8, num_blocks=n_req * 8,
                                                                    max_batch_size=n_req, dtype=dtype))
    got = engine.generate(prompts, [SamplingParams(max_tokens=n, temperature=0.0) for n in news])
    assert engine.stats()["graph_steps"] > 0
    assert engine.cache.num_free_pages() == n_req * 8 and engine.cache.check() == 0
    exact = 0
    for prompt, tokens, n in zip(prompts, got, news):
        assert len(tokens) == n
        exact += _assert_greedy_within_tolerance(model_folders["B"], prompt, tokens, dtype)
    if dtype == "float32":
        assert exact == sum(news)
    else:
        assert exact >= 0.9 * sum(news)


@pytest.mark.parametrize("shape,n_req", [("50M", 8), ("50M", 3), ("small", 20), ("xl", 64), ("xl", 256), ("50M", 200)])
def test_real_widths_decode_through_graphs_and_bursts(tmp_path, shape, n_req):
    """The benchmarked shapes through the engine itself (padded graphs, bursts of steps fed on the
    device): every greedy choice is the plain implementation's argmax up to the logits' tolerance.
    The runs of 200 and 256 requests (the capacity-256 graph, whose products go to the tiled kernels)
    have a page pool that does not hold everybody's last tokens: requests are evicted and recomputed
    (the reference's tests of its paged engine against its oracle, tests/test_paged.py:45-143)."""
    from mini_gpt_inference_amd import GPTConfig
    from mini_gpt_inference_amd.weights.random_init import write_random_model
    family = {"50M": dict(n_layer=2, n_embd=512, n_head=8, vocab_size=50304),
              "small": dict(n_layer=1, n_embd=768, n_head=12, vocab_size=50257),
              "xl": dict(n_layer=1, n_embd=1600, n_head=25, vocab_size=50257)}[shape]
    cfg = GPTConfig("gpt2-mini", block_size=64, bias=True, layer_norm_eps=1e-5, **family)
    folder = write_random_model(str(tmp_path / shape), cfg, 11, std_scale=3.0)
    rng = np.random.default_rng(n_req)
    prompts = [helpers.random_ids(rng, cfg.vocab_size, int(n)) for n in rng.integers(1, 9, n_req)]
    n_new = 20
    tight = n_req >= 200
    engine = LLMEngine.from_folder(folder, EngineConfig(block_size=16, num_blocks=n_req * 2 - (n_req // 3 if tight else 0),
                                                        max_batch_size=n_req, dtype="bfloat16"))
    got = engine.generate(prompts, SamplingParams(max_tokens=n_new, temperature=0.0))
    assert engine.stats()["graph_steps"] >= n_new - 4
    assert (engine.stats()["num_preemptions"] > 0) == tight
    assert engine.cache.check() == 0 and engine.cache.num_free_pages() == engine.cache.groups[0].num_pages
    # up to 16 rows of a vocabulary of whole tiles choose from the bests that the head leaves per tile
    assert all(g.tile_best_used == (shape == "50M" and g.cap <= 16) for g in engine._graphs.values() if g.graph)
    pcfg, w = P.read_model_folder(folder)
    exact = total = 0
    for prompt, tokens in list(zip(prompts, got))[::max(1, n_req // 8)]:      # a sample of the requests: the plain model is slow
        assert len(tokens) == n_new
        ids = list(prompt)
        for tok in tokens:
            logits = P.plain_forward(w, pcfg, ids, rows=[len(ids) - 1])[0].numpy()
            assert logits[tok] >= logits.max() - 2 * helpers.TOL["bfloat16"] * max(1.0, np.abs(logits).max())
            exact += tok == int(np.argmax(logits))
            total += 1
            ids.append(tok)
    assert exact >= 0.9 * total


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", range(6))
def test_drawn_configurations_generate_through_graphs_and_bursts(tmp_path, seed, dtype):
    """Configurations drawn from a seed (every size and option varies), a drawn number of requests:
    greedy generation through the entry point, its decode steps from graphs and bursts (and, in
    bfloat16 at widths that take them, the fused kernels), gives the plain implementation's tokens."""
    from safetensors.torch import save_file
    from mini_gpt_inference_amd.config.model_config import write_config_json
    from mini_gpt_inference_amd.weights.random_init import random_tensors
    from test_gpu_replay import _drawn_configuration
    cfg = _drawn_configuration(seed + 20)
    folder = str(tmp_path / f"drawn{seed}")
    os.makedirs(folder)
    write_config_json(folder, cfg)
    save_file({k: v.contiguous() for k, v in random_tensors(cfg, seed, torch.bfloat16, 4.0).items()},
              os.path.join(folder, "model.safetensors"))
    rng = np.random.default_rng(seed)
    n_req, n_new = int(rng.integers(1, 10)), 20
    prompts = [helpers.random_ids(rng, cfg.vocab_size, int(n)) for n in rng.integers(1, cfg.block_size - n_new, n_req)]
    page = int(rng.choice([4, 8, 16]))
    pages = n_req * (-(-cfg.block_size // page))
    engine = LLMEngine.from_folder(folder, EngineConfig(block_size=page, num_blocks=pages, max_batch_size=n_req,
                                                        dtype=dtype))
    got = engine.generate(prompts, SamplingParams(max_tokens=n_new, temperature=0.0))
    assert engine.stats()["graph_steps"] >= n_new - 4
    assert engine.cache.check() == 0 and engine.cache.num_free_pages() == pages
    if dtype == "float32":
        assert got == _plain_greedy(folder, prompts, n_new)
    else:
        for prompt, tokens in zip(prompts, got):
            assert len(tokens) == n_new
            _assert_greedy_within_tolerance(folder, prompt, tokens, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_chunked_mixed_and_whole_prompt_policies_give_the_same_tokens(model_folders, dtype):
    prompts = _prompts("B", [1, 9, 33, 64, 100], seed=2)
    sp = SamplingParams(max_tokens=16, temperature=0.0)
    outs = []
    for kw in (dict(prefill_chunk=0, mixed_batches=False), dict(prefill_chunk=16, mixed_batches=True),
               dict(prefill_chunk=7, max_num_batched_tokens=24, mixed_batches=True, use_graph=False)):
        engine = LLMEngine.from_folder(model_folders["B"], EngineConfig(block_size=8, num_blocks=96, max_batch_size=4,
                                                                        dtype=dtype, **kw))
        outs.append(engine.generate(prompts, sp))
    if dtype == "float32":
        assert outs[0] == outs[1] == outs[2]
    else:   # bfloat16 kernels differ between few and many rows: each choice is the argmax up to rounding
        for out in outs:
            for prompt, tokens in zip(prompts, out):
                _assert_greedy_within_tolerance(model_folders["B"], prompt, tokens, dtype)


def test_seeded_temperature_sampling_is_reproducible_and_independent_of_batching(model_folders):
    # The family's second tiny workload: five requests of 1/9/33/64/100 tokens, 16 tokens at temperature 0.8 from a
    # fixed sampler seed, prompt portions of 16, pages of 8
    prompts = _prompts("B", [1, 9, 33, 64, 100], seed=3)
    params = [SamplingParams(max_tokens=16, temperature=0.8, seed=100 + i) for i in range(5)]

    def run(**kw):
        cfg = EngineConfig(block_size=8, num_blocks=128, dtype="float32", seed=7, **kw)
        return LLMEngine.from_folder(model_folders["B"], cfg).generate(prompts, params)

    together = run(max_batch_size=8, prefill_chunk=16)
    assert together == run(max_batch_size=8, prefill_chunk=16)
    assert together == run(max_batch_size=2, prefill_chunk=0, mixed_batches=False)    # other batches, same tokens
    assert together != LLMEngine.from_folder(model_folders["B"], EngineConfig(
        block_size=8, num_blocks=128, dtype="float32", seed=8)).generate(prompts, params)
    # each token is the plain sampler's choice for the plain logits and the same uniform number
    cfg, w = P.read_model_folder(model_folders["B"])
    for i in (0, 2):
        ids = list(prompts[i])
        for k, tok in enumerate(together[i][:6]):
            logits = P.plain_forward(w, cfg, ids)[-1].numpy()
            u = P.plain_uniform(7, 100 + i, k)
            want, lo, hi, total = P.plain_sample(logits, 0.8, None, None, u)
            assert tok == want or min(abs(u * total - lo), abs(u * total - hi)) < 1e-3 * total
            ids.append(tok)


@pytest.mark.parametrize("evict", ["newest", "newest_other"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_pages_run_out_preempted_request_is_recomputed_and_ends_with_the_same_tokens(model_folders, dtype, evict):
    # reference tests/test_paged.py:107-143: pages of 2, four pages, two prompts of 2, 4 new tokens each
    prompts = [[1, 2], [4, 5]]
    sp = SamplingParams(max_tokens=4, temperature=0.0)
    roomy = LLMEngine.from_folder(model_folders["A"], EngineConfig(block_size=2, num_blocks=64, max_batch_size=2,
                                                                   dtype=dtype)).generate(prompts, sp)
    engine = LLMEngine.from_folder(model_folders["A"], EngineConfig(block_size=2, num_blocks=4, max_batch_size=2,
                                                                    dtype=dtype, evict=evict))
    tight = engine.generate(prompts, sp)
    assert engine.stats()["num_preemptions"] > 0
    assert engine.cache.num_free_pages() == 4 and engine.cache.check() == 0
    if dtype == "float32":
        assert tight == roomy == _plain_greedy(model_folders["A"], prompts, 4)
    else:
        for prompt, tokens in zip(prompts, tight):
            _assert_greedy_within_tolerance(model_folders["A"], prompt, tokens, dtype)


def test_fragmentation_stats_follow_the_requests(model_folders):
    # src/minigpt_infer/cache/paged.py:83-94: free, allocated, and slots allocated beyond the computed tokens
    engine = LLMEngine.from_folder(model_folders["A"], EngineConfig(block_size=4, num_blocks=32, max_batch_size=4,
                                                                    decode_burst=1, dtype="float32"))
    assert engine.fragmentation_stats() == {"free_blocks": 32, "allocated_blocks": 0,
                                            "internal_fragmentation_slots": 0}
    engine.add_request(Request("a", [1, 2, 3, 4, 5], SamplingParams(max_tokens=6, temperature=0.0)))
    engine.add_request(Request("b", [7], SamplingParams(max_tokens=3, temperature=0.0)))
    engine.step()      # both prompts: 5 and 1 tokens computed, pages for 5 and 1 tokens
    assert engine.fragmentation_stats() == {"free_blocks": 29, "allocated_blocks": 3,
                                            "internal_fragmentation_slots": 3 * 4 - 6}
    engine.step()      # one decoded token each: 6 and 2 computed
    assert engine.fragmentation_stats()["internal_fragmentation_slots"] == 3 * 4 - 8
    while engine.has_unfinished_requests():
        engine.step()
    assert engine.fragmentation_stats() == {"free_blocks": 32, "allocated_blocks": 0,
                                            "internal_fragmentation_slots": 0}


def test_step_outputs_finish_reasons_eot_and_cancel(model_folders):
    engine = LLMEngine.from_folder(model_folders["A"], EngineConfig(block_size=4, num_blocks=32, max_batch_size=4,
                                                                    dtype="float32"))
    # a prompt whose greedy continuation changes token somewhere, so that an end token can be told apart
    for seed in range(20):
        prompt = _prompts("A", [7], seed=seed)[0]
        first = _plain_greedy(model_folders["A"], [prompt], 8)[0]
        k = next((i for i, t in enumerate(first) if t not in first[:i] and i > 0), None)
        if k is not None:
            break
    assert k is not None
    engine.add_request(Request("len", prompt, SamplingParams(max_tokens=2, temperature=0.0)))
    engine.add_request(Request("eot", prompt, SamplingParams(max_tokens=20, temperature=0.0), eot_token_id=first[k]))
    engine.add_request(Request("gone", prompt, SamplingParams(max_tokens=20, temperature=0.0)))
    seen = {}
    steps = 0
    while engine.has_unfinished_requests():
        for out in engine.step():
            assert len(out.new_token_ids) == 1      # one token per request and step (reference engine.py:177-183)
            seen.setdefault(out.request_id, []).append(out)
        steps += 1
        if steps == 1:
            assert engine.cancel_request("gone") and not engine.cancel_request("nobody")
    assert [o.new_token_ids[0] for o in seen["len"]] == first[:2] and seen["len"][-1].finish_reason == "length"
    assert [o.new_token_ids[0] for o in seen["eot"]] == first[:k + 1] and seen["eot"][-1].finish_reason == "eot"
    assert len(seen["gone"]) == 1 and not seen["gone"][0].finished
    assert engine.cache.num_free_pages() == 32
    with pytest.raises(SchedulerError, match="block_size"):          # reference engine.py:83-88
        engine.add_request(Request("long", list(range(60)), SamplingParams(max_tokens=10)))
    with pytest.raises(ValueError, match="token id"):
        engine.add_request(Request("bad", [1, 999], SamplingParams(max_tokens=2)))


def test_finished_requests_are_forgotten_and_their_ids_can_be_used_again(model_folders):
    engine = LLMEngine.from_folder(model_folders["A"], EngineConfig(block_size=4, num_blocks=64, max_batch_size=4,
                                                                    dtype="float32"))
    prompts = _prompts("A", [5, 9], seed=12)
    first = engine.generate(prompts, SamplingParams(max_tokens=5, temperature=0.0))
    assert not engine._ids and not engine._rids          # generate() leaves nothing behind
    assert engine.generate(prompts, SamplingParams(max_tokens=5, temperature=0.0)) == first
    engine.add_request(Request("mine", prompts[0], SamplingParams(max_tokens=3, temperature=0.0)))
    with pytest.raises(ValueError):
        engine.add_request(Request("mine", prompts[1], SamplingParams(max_tokens=3, temperature=0.0)))
    while engine.has_unfinished_requests():
        engine.step()
    assert engine.forget_finished() == 1 and engine.forget_finished() == 0
    engine.add_request(Request("mine", prompts[1], SamplingParams(max_tokens=3, temperature=0.0)))
    got = []
    while engine.has_unfinished_requests():
        got += [t for out in engine.step() for t in out.new_token_ids]
    assert got == first[1][:3]
    assert engine.cache.num_free_pages() == 64 and engine.cache.check() == 0


def test_requests_that_end_while_the_next_chain_is_already_enqueued(model_folders):
    """An end token met in a chain's last steps: the chain enqueued behind it computes for requests
    that are over; its tokens are dropped, and the engine goes on with whoever comes next."""
    prompts = _prompts("B", [7, 12], seed=40)
    plain = _plain_greedy(model_folders["B"], prompts, 30)
    engine = LLMEngine.from_folder(model_folders["B"], EngineConfig(block_size=8, num_blocks=64, max_batch_size=4,
                                                                    dtype="float32", decode_burst=2, decode_chain=2))
    # request 0 ends by its end token some chains in (further steps are planned ahead by then),
    # request 1 is cancelled by the caller at that moment
    first = [j for j in range(4, 30) if plain[0][j] not in plain[0][:j]]
    assert first, "the plain tokens never bring a new token: choose another seed"
    eot = plain[0][first[0]]
    engine.add_request(Request("a", prompts[0], SamplingParams(max_tokens=30, temperature=0.0), eot_token_id=eot))
    engine.add_request(Request("b", prompts[1], SamplingParams(max_tokens=30, temperature=0.0)))
    got = {"a": [], "b": []}
    while "a" in engine._rids and engine.scheduler.info(engine._rids["a"]).status != 2:
        for out in engine.step():
            got[out.request_id] += out.new_token_ids
    assert got["a"] == plain[0][:first[0] + 1]
    engine.cancel_request("b")
    assert not engine.has_unfinished_requests()
    assert got["b"] == plain[1][:len(got["b"])]
    # the engine is used again while a chain for the two is still enqueued
    again = engine.generate(prompts, SamplingParams(max_tokens=9, temperature=0.0))
    assert again == [p[:9] for p in plain]
    assert engine.cache.num_free_pages() == 64 and engine.cache.check() == 0 and engine._inflight is None


def test_decode_graphs_can_be_captured_before_the_first_request(model_folders):
    prompts = _prompts("A", [5, 17, 30])
    want = _plain_greedy(model_folders["A"], prompts, 12)
    engine = LLMEngine.from_folder(model_folders["A"], EngineConfig(block_size=4, num_blocks=96, max_batch_size=4,
                                                                    dtype="float32"))
    assert engine.capture_decode_graphs() == [1, 2, 4]
    assert engine.cache.num_free_pages() == 96 and engine.cache.check() == 0 and not engine._rids
    graphs = {cap: (g.graph, g.burst_graph) for cap, g in engine._graphs.items()}
    assert all(g is not None and b is not None for g, b in graphs.values())
    eager_before = engine.stats()["eager_steps"]
    assert engine.generate(prompts, SamplingParams(max_tokens=12, temperature=0.0)) == want
    # nothing was captured again, and only the prompts' step ran outside a decode graph
    assert {cap: (g.graph, g.burst_graph) for cap, g in engine._graphs.items()} == graphs
    assert engine.stats()["eager_steps"] - eager_before == 1
    # too few pages for four made-up requests: that capacity is left out
    small = LLMEngine.from_folder(model_folders["A"], EngineConfig(block_size=4, num_blocks=20, max_batch_size=4,
                                                                   dtype="float32"))
    assert small.capture_decode_graphs() == [1, 2]
    with pytest.raises(RuntimeError):
        small.add_request(Request("x", [1, 2], SamplingParams(max_tokens=4)))
        small.capture_decode_graphs()


def test_stats_count_the_weights_and_the_copies_made_of_them(model_folders):
    """stats() reports the bytes of the tensors as loaded (the tied head once) and of the copies the
    kernels made of the matrices at first use, which are none before the first step."""
    cfg = helpers.CONFIGS["A"]
    engine = LLMEngine.from_folder(model_folders["A"], EngineConfig(block_size=4, num_blocks=32, max_batch_size=2,
                                                                    dtype="bfloat16"))
    c, f, v, p, L = cfg.n_embd, 4 * cfg.n_embd, cfg.vocab_size, cfg.block_size, cfg.n_layer
    matrices = (v * c + p * c + L * (3 * c * c + c * c + 2 * f * c)) * 2
    vectors = ((2 * L + 1) * 2 * c + L * (3 * c + c + f + c)) * 4
    before = engine.stats()
    assert before["weight_bytes"] == matrices + vectors and before["derived_weight_bytes"] == 0
    assert before["cache_bytes"] == L * 2 * 32 * cfg.n_head * 4 * cfg.head_dim * 2
    engine.generate([[1, 2, 3]], SamplingParams(max_tokens=4, temperature=0.0))
    after = engine.stats()
    assert after["weight_bytes"] == before["weight_bytes"]
    # every matrix of the layers has at least its packed copy by now
    assert after["derived_weight_bytes"] >= L * (3 * c * c + c * c + 2 * f * c) * 2


@pytest.mark.parametrize("limit", [0, 40_000])
def test_the_copies_of_matrices_stay_within_their_bound(model_folders, limit):
    """EngineConfig.derived_weight_bytes bounds the copies that the decode kernels make of matrices
    at first use (0: none at all): the matrices whose copies do not fit are read as loaded, and the
    tokens are still the plain implementation's argmax up to rounding."""
    prompts = _prompts("B", [9, 33, 2], seed=6)
    engine = LLMEngine.from_folder(model_folders["B"], EngineConfig(block_size=8, num_blocks=64, max_batch_size=4,
                                                                    dtype="bfloat16", derived_weight_bytes=limit))
    got = engine.generate(prompts, SamplingParams(max_tokens=10, temperature=0.0))
    stats = engine.stats()
    assert stats["derived_weight_bytes"] <= limit and (limit == 0 or stats["derived_weight_bytes"] > 0)
    assert stats["graph_steps"] > 0
    for prompt, tokens in zip(prompts, got):
        _assert_greedy_within_tolerance(model_folders["B"], prompt, tokens, "bfloat16")
    free = LLMEngine.from_folder(model_folders["B"], EngineConfig(block_size=8, num_blocks=64, max_batch_size=4,
                                                                  dtype="bfloat16"))
    free.generate(prompts, SamplingParams(max_tokens=10, temperature=0.0))
    assert free.stats()["derived_weight_bytes"] > 40_000


def test_real_vocabulary_bound_is_never_crossed(model_folders):
    engine = LLMEngine.from_folder(model_folders["A"], EngineConfig(block_size=4, num_blocks=32, max_batch_size=4,
                                                                    dtype="float32", real_vocab_size=40))
    outs = engine.generate(_prompts("A", [6, 9]), SamplingParams(max_tokens=10, temperature=1.5, seed=1))
    assert all(t < 40 for o in outs for t in o)


def test_from_random_and_the_command_line(tmp_path, model_folders):
    cfg = helpers.CONFIGS["A"]
    a = LLMEngine.from_random(cfg, 3, EngineConfig(dtype="float32", num_blocks=32, max_batch_size=2))
    b = LLMEngine.from_random(cfg, 3, EngineConfig(dtype="float32", num_blocks=32, max_batch_size=2))
    sp = SamplingParams(max_tokens=5, temperature=0.0)
    assert a.generate([[1, 2, 3]], sp) == b.generate([[1, 2, 3]], sp)
    want = _plain_greedy(model_folders["A"], [[5, 17, 3, 200]], 6)[0]
    proc = subprocess.run([sys.executable, "-m", "mini_gpt_inference_amd.generate", "--model", model_folders["A"],
                           "--prompt-ids", "5,17,3,200", "--max-new-tokens", "6", "--temperature", "0",
                           "--dtype", "float32", "--kv-block-size", "4", "--num-kv-blocks", "32"],
                          cwd=ROOT, capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert "config: GPTConfig(" in proc.stdout
    line = next(l for l in proc.stdout.splitlines() if l.startswith("sample:"))
    assert [int(t) for t in line.split()[1:]] == want


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_bursts_change_nothing_but_the_pace(model_folders, dtype):
    """Steps enqueued back to back with tokens fed on the device give the tokens that one step at a
    time gives: greedy and seeded, with an end token met inside a burst; also with several bursts
    enqueued before the host waits, whose tokens are taken in while the device runs the next, and
    with the next chain enqueued before the last tokens of this one are in."""
    prompts = _prompts("B", [3, 20, 41], seed=6)
    plain_first = _plain_greedy(model_folders["B"], prompts[:1], 12)[0]
    eot = plain_first[6]
    params = [SamplingParams(max_tokens=24, temperature=0.0), SamplingParams(max_tokens=17, temperature=0.9, seed=5),
              SamplingParams(max_tokens=24, temperature=0.7, top_k=20, seed=6)]
    outs, steps = [], []
    for burst, chain, ahead in ((1, 1, False), (8, 1, False), (4, 3, False), (2, 4, True), (2, 1, True), (8, 2, True)):
        engine = LLMEngine.from_folder(model_folders["B"], EngineConfig(block_size=8, num_blocks=64, max_batch_size=4,
                                                                        dtype=dtype, decode_burst=burst,
                                                                        decode_chain=chain, decode_ahead=ahead, seed=3))
        for i, (p, sp) in enumerate(zip(prompts, params)):
            engine.add_request(Request(f"r{i}", p, sp, eot_token_id=eot if i == 0 else None))
        got = {f"r{i}": [] for i in range(3)}
        calls = 0
        while engine.has_unfinished_requests():
            for out in engine.step():
                got[out.request_id] += out.new_token_ids
            calls += 1
        outs.append(got)
        steps.append(calls)
        assert engine.cache.num_free_pages() == 64 and engine.cache.check() == 0
    assert all(o == outs[0] for o in outs[1:])
    assert max(steps[1:]) < steps[0]                # the bursts were taken
    if dtype == "float32":
        assert outs[0]["r0"] == plain_first[:plain_first.index(eot) + 1]


@pytest.mark.parametrize("name,seed", [("A", 0), ("A", 1), ("A", 2), ("A", 3), ("B", 4), ("B", 5), ("B", 6), ("B", 7),
                                       ("C", 8), ("D", 9)])
def test_random_engine_settings_give_the_tokens_of_one_step_at_a_time_32bit(model_folders, name, seed):
    """Sampled and greedy requests with end tokens arrive over time; an engine with drawn settings
    (page pool, batch size, token budget, portions, bursts, chains, steps enqueued ahead) gives every
    request the tokens that an engine without bursts and with room for everything gives it."""
    cfg = helpers.CONFIGS[name]
    rng = np.random.default_rng(5000 + seed)
    reqs = []
    for i in range(int(rng.integers(6, 20))):
        n = int(rng.integers(1, cfg.block_size // 2))
        m = int(rng.integers(2, min(40, cfg.block_size - n)))
        t = float(rng.choice([0.0, 0.7, 1.3]))
        sp = SamplingParams(max_tokens=m, temperature=t, top_k=int(rng.integers(0, 30)) or None,
                            top_p=float(rng.choice([1.0, 0.9, 0.5])) if t > 0 else None, seed=int(rng.integers(0, 1000)))
        eot = int(rng.integers(0, cfg.vocab_size)) if rng.random() < 0.7 else None
        reqs.append((helpers.random_ids(rng, cfg.vocab_size, n), sp, eot))
    arrivals = sorted((int(rng.integers(0, 30)), i) for i in range(len(reqs)))
    page = 4
    pool = max(-(-(len(p) + sp.max_tokens) // page) for p, sp, _ in reqs) + int(rng.integers(2, 60))

    def run(ecfg):
        engine = LLMEngine.from_folder(model_folders[name], ecfg)
        got = {i: [] for i in range(len(reqs))}
        todo, step = list(arrivals), 0
        while todo or engine.has_unfinished_requests():
            while todo and todo[0][0] <= step:
                _, i = todo.pop(0)
                engine.add_request(Request(f"r{i}", reqs[i][0], reqs[i][1], eot_token_id=reqs[i][2]))
            for out in engine.step():
                got[int(out.request_id[1:])].extend(out.new_token_ids)
            step += 1
            if step % 7 == 0:
                engine.forget_finished()
            assert step < 5000, "the engine makes no progress"
        engine.step(max_decode_steps=0)      # steps enqueued ahead for requests that ended since
        assert engine.cache.check() == 0 and engine.cache.num_free_pages() == ecfg.num_blocks
        return got

    base = run(EngineConfig(block_size=page, num_blocks=pool + 50, max_batch_size=4, dtype="float32", decode_burst=1, seed=9))
    drawn = EngineConfig(block_size=page, num_blocks=pool, max_batch_size=int(rng.integers(1, 24)),
                         max_num_batched_tokens=int(rng.integers(8, 64)), prefill_chunk=int(rng.integers(0, 12)),
                         dtype="float32", decode_burst=int(rng.integers(2, 9)), decode_chain=int(rng.integers(1, 5)),
                         decode_ahead=True, seed=9)
    assert run(drawn) == base, drawn


@pytest.mark.parametrize("name,seed", [("A", 0), ("B", 1), ("C", 2)])
def test_arrivals_evictions_bursts_and_cancels_together_32bit(model_folders, name, seed):
    """Requests arrive while others decode, the page pool is too small for all of them, prompts are
    cut into portions, decode steps run in bursts, one request is cancelled on the way: every
    request that ends has exactly the plain implementation's greedy tokens, and nothing is left
    allocated."""
    cfg = helpers.CONFIGS[name]
    rng = np.random.default_rng(100 + seed)
    n_req = 9
    lens = [int(rng.integers(1, cfg.block_size // 2)) for _ in range(n_req)]
    news = [int(rng.integers(3, min(24, cfg.block_size - n))) for n in lens]
    prompts = [helpers.random_ids(rng, cfg.vocab_size, n) for n in lens]
    page = 4
    worst = max(-(-(n + m) // page) for n, m in zip(lens, news))
    engine = LLMEngine.from_folder(model_folders[name], EngineConfig(
        block_size=page, num_blocks=worst + 6, max_batch_size=4, max_num_batched_tokens=24, prefill_chunk=7,
        dtype="float32", decode_burst=4))
    got = {i: [] for i in range(n_req)}
    arrivals = sorted((int(rng.integers(0, 25)), i) for i in range(n_req))
    cancelled, step = None, 0
    while arrivals or engine.has_unfinished_requests():
        while arrivals and arrivals[0][0] <= step:
            _, i = arrivals.pop(0)
            engine.add_request(Request(f"r{i}", prompts[i], SamplingParams(max_tokens=news[i], temperature=0.0)))
        if step == 12 and cancelled is None:
            live = [i for i in range(n_req) if f"r{i}" in engine._rids and len(got[i]) < news[i]]
            if live:
                cancelled = live[-1]
                engine.cancel_request(f"r{cancelled}")
        for out in engine.step():
            got[int(out.request_id[1:])].extend(out.new_token_ids)
        step += 1
        assert step < 2000, "the engine makes no progress"
    want = _plain_greedy(model_folders[name], prompts, max(news))
    for i in range(n_req):
        if i == cancelled:
            assert got[i] == want[i][:len(got[i])]
        else:
            assert got[i] == want[i][:news[i]], f"request {i}"
    stats = engine.stats()
    assert stats["free_blocks"] == worst + 6 and engine.cache.check() == 0
    # with these draws every configuration evicts, replays graphs and runs eager (prompt) steps
    assert stats["num_preemptions"] > 0 and stats["graph_steps"] > 0 and stats["eager_steps"] > 0

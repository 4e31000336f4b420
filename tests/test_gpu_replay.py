"""Trace replay against the plain implementation: the same requests whole, with the last 32
tokens one by one, in portions of changing size, and mixed with page reuse; in 32-bit and in
bfloat16; through the replay class and through bin/trace_run itself."""

import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import helpers
import plain_gpt as P
from mini_gpt_inference_amd.engine.replay import TraceError, TraceReplayer

pytestmark = pytest.mark.gpu

LENGTHS = {"A": [5, 17, 30, 64, 41, 23], "B": [1, 9, 33, 64, 100, 128], "C": [2, 96, 40, 71, 18],
           "D": [200, 3, 130, 77, 150], "E": [72, 5, 40, 33, 64], "F": [3, 80, 47, 66, 21]}


def _requests(name, rng):
    cfg = helpers.CONFIGS[name]
    return {f"r{i}": helpers.random_ids(rng, cfg.vocab_size, n) for i, n in enumerate(LENGTHS[name])}


_plain_cache = {}


def _plain_logits(folder, name, reqs):
    key = (name, tuple(map(tuple, reqs.values())))
    if key not in _plain_cache:
        cfg, w = P.read_model_folder(folder)
        _plain_cache[key] = {rid: P.plain_forward(w, cfg, ids).numpy() for rid, ids in reqs.items()}
    return _plain_cache[key]


@pytest.mark.parametrize("page_size", [16, 4])
@pytest.mark.parametrize("way", ["whole", "tail", "portions", "mixed"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_every_way_of_cutting_matches_the_plain_implementation(model_folders, name, dtype, way, page_size):
    rng = np.random.default_rng(11)
    reqs = _requests(name, rng)
    want = _plain_logits(model_folders[name], name, reqs)
    plan = helpers.PLANS[way](reqs, np.random.default_rng(5))
    # the pool holds just what the live requests need, so freed pages are used again;
    # it starts as NaN, so a read of a slot nobody wrote shows
    replayer = TraceReplayer(model_folders[name], dtype, plan.tight_tokens(page_size), page_size=page_size,
                             poison=True)
    got = plan.assemble(helpers.run_plan_in_process(replayer, plan), {r: len(t) for r, t in reqs.items()},
                        helpers.CONFIGS[name].vocab_size)
    for rid in reqs:
        helpers.assert_close(got[rid], want[rid], dtype, f"{name} {dtype} {way} {rid}")
    assert replayer.cache.check() == 0
    assert replayer.cache.num_free_pages() == replayer.num_pages and not replayer.live
    if way == "mixed":
        total = sum(-(-len(t) // page_size) for t in reqs.values())
        assert total > replayer.num_pages, "the pool is so large that no page was used twice"


@pytest.mark.parametrize("way", ["whole", "tail", "portions", "mixed"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["C", "D"])
def test_head_sizes_that_are_no_power_of_two(model_folders, name, dtype, way):
    """Head sizes 48 and 80 and widths 144 and 80: the kernels that only take some head sizes must
    hand over to the general ones, never compute something else."""
    reqs = _requests(name, np.random.default_rng(17))
    want = _plain_logits(model_folders[name], name, reqs)
    plan = helpers.PLANS[way](reqs, np.random.default_rng(6))
    replayer = TraceReplayer(model_folders[name], dtype, plan.tight_tokens(16), poison=True)
    got = plan.assemble(helpers.run_plan_in_process(replayer, plan), {r: len(t) for r, t in reqs.items()},
                        helpers.CONFIGS[name].vocab_size)
    for rid in reqs:
        helpers.assert_close(got[rid], want[rid], dtype, f"{name} {dtype} {way} {rid}")
    assert replayer.cache.check() == 0 and replayer.cache.num_free_pages() == replayer.num_pages


@pytest.mark.parametrize("way", ["whole", "tail", "portions", "mixed"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["E", "F"])
def test_head_sizes_and_widths_that_are_no_multiple_of_16(model_folders, name, dtype, way):
    """n_embd 40 with one head and n_embd 36 with three heads of 12: the architecture takes any width
    that the heads divide (src/minigpt_infer/model.py:39-41).  The matrix-core kernels refuse such
    inner sizes and head sizes; the general kernels take them, in both dtypes, cut in every way."""
    reqs = _requests(name, np.random.default_rng(19))
    want = _plain_logits(model_folders[name], name, reqs)
    plan = helpers.PLANS[way](reqs, np.random.default_rng(7))
    replayer = TraceReplayer(model_folders[name], dtype, plan.tight_tokens(8), page_size=8, poison=True)
    got = plan.assemble(helpers.run_plan_in_process(replayer, plan), {r: len(t) for r, t in reqs.items()},
                        helpers.CONFIGS[name].vocab_size)
    for rid in reqs:
        helpers.assert_close(got[rid], want[rid], dtype, f"{name} {dtype} {way} {rid}")
    assert replayer.cache.check() == 0 and replayer.cache.num_free_pages() == replayer.num_pages


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_logit_rows_of_a_decode_step_in_any_order(model_folders, dtype):
    """A decode-only step whose wanted rows are as many as its tokens but not 0, 1, 2 in order (a
    permutation, a row twice): the logits come in the order asked for, also when the same shape
    came before with the rows in order (whose graph or plan drops the row list)."""
    cfg = helpers.CONFIGS["A"]
    rng = np.random.default_rng(31)
    seqs = [helpers.random_ids(rng, cfg.vocab_size, n) for n in (12, 14, 11)]
    pcfg, w = P.read_model_folder(model_folders["A"])
    want = [P.plain_forward(w, pcfg, s).numpy() for s in seqs]
    rep = TraceReplayer(model_folders["A"], dtype, 256, poison=True)
    slots = [rep.cache.acquire_slot() for _ in seqs]
    for slot, s in zip(slots, seqs):
        assert rep.cache.reserve(slot, len(s))
    heads = [3, 5, 2]
    rep.runner.step(slots, [0, 0, 0], heads, sum((s[:h] for s, h in zip(seqs, heads)), []), [])
    for j, rows in enumerate([[0, 1, 2], [0, 1, 2], [0, 1, 2], [0, 1, 2], [2, 0, 1], [1, 1, 0], [0, 1, 2], [2, 2, 2]]):
        ctx = [h + j for h in heads]
        got = rep.runner.step(slots, ctx, [1, 1, 1], [s[c] for s, c in zip(seqs, ctx)], rows).cpu()
        ref = np.stack([want[r][ctx[r]] for r in rows])
        helpers.assert_close(got, ref, dtype, f"step {j}, rows {rows}")
    assert rep.runner.num_replayed_steps >= 1


def _drawn_configuration(seed):
    """A configuration drawn from the seed: every size and option of the architecture varies."""
    from mini_gpt_inference_amd import GPTConfig
    rng = np.random.default_rng(1000 + seed)
    head = int(rng.choice([16, 32, 48, 64, 80, 128]))
    heads = int(rng.integers(1, 7 if head <= 64 else 4))
    return GPTConfig("gpt2-mini", n_layer=int(rng.integers(1, 4)), n_embd=head * heads, n_head=heads,
                     vocab_size=int(rng.integers(50, 700)), block_size=int(rng.choice([64, 96, 160, 256])),
                     bias=bool(rng.integers(0, 2)), layer_norm_eps=float(rng.choice([1e-6, 1e-5, 1e-3])))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", range(8))
def test_drawn_configurations_mixed_with_page_reuse(tmp_path, seed, dtype):
    """Configurations nobody chose by hand (head sizes 16 to 128, one to six heads, any vocabulary,
    with and without biases), requests of drawn lengths, mixed steps, a tight poisoned pool of drawn
    page size: whichever kernels the sizes select, the logits are the plain implementation's."""
    from safetensors.torch import save_file
    from mini_gpt_inference_amd.config.model_config import write_config_json
    from mini_gpt_inference_amd.weights.random_init import random_tensors
    cfg = _drawn_configuration(seed)
    folder = str(tmp_path / f"drawn{seed}")
    os.makedirs(folder)
    write_config_json(folder, cfg)
    save_file({k: v.contiguous() for k, v in random_tensors(cfg, seed, torch.bfloat16, 4.0).items()},
              os.path.join(folder, "model.safetensors"))
    rng = np.random.default_rng(seed)
    page_size = int(rng.choice([2, 4, 8, 16, 32]))
    lengths = [int(n) for n in rng.integers(1, cfg.block_size + 1, 5)]
    reqs = {f"r{i}": helpers.random_ids(rng, cfg.vocab_size, n) for i, n in enumerate(lengths)}
    pcfg, w = P.read_model_folder(folder)
    plan = helpers.plan_mixed(reqs, np.random.default_rng(seed + 50))
    replayer = TraceReplayer(folder, dtype, plan.tight_tokens(page_size), page_size=page_size, poison=True)
    got = plan.assemble(helpers.run_plan_in_process(replayer, plan), {r: len(t) for r, t in reqs.items()},
                        cfg.vocab_size)
    for rid, ids in reqs.items():
        helpers.assert_close(got[rid], P.plain_forward(w, pcfg, ids).numpy(), dtype, f"{cfg} {dtype} {rid}")
    assert replayer.cache.check() == 0 and replayer.cache.num_free_pages() == replayer.num_pages


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_cuts_agree_with_each_other_bit_for_bit_in_32_bit(model_folders, dtype):
    """On the 32-bit path the order of every sum depends only on a token's position, so all ways of
    cutting give identical logits, not merely close ones."""
    rng = np.random.default_rng(3)
    reqs = _requests("A", rng)
    results = []
    for way in ("whole", "tail", "portions", "mixed"):
        plan = helpers.PLANS[way](reqs, np.random.default_rng(9))
        replayer = TraceReplayer(model_folders["A"], dtype, plan.max_tokens, poison=True)
        results.append(plan.assemble(helpers.run_plan_in_process(replayer, plan),
                                     {r: len(t) for r, t in reqs.items()}, helpers.CONFIGS["A"].vocab_size))
    for other in results[1:]:
        for rid in reqs:
            if dtype == "float32":
                assert np.array_equal(results[0][rid], other[rid])
            else:
                helpers.assert_close(other[rid], results[0][rid], dtype, rid)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(model_folders, tmp_path, dtype):
    """bin/trace_run itself: all four ways in one session, files and `done` lines as specified."""
    name = "B"
    rng = np.random.default_rng(21)
    cfg = helpers.CONFIGS[name]
    reqs = {f"q{i}": helpers.random_ids(rng, cfg.vocab_size, n) for i, n in enumerate([3, 40, 77, 128, 65])}
    want = _plain_logits(model_folders[name], name, reqs)
    plans = [helpers.PLANS[w](reqs, np.random.default_rng(2)) for w in ("whole", "tail", "portions", "mixed")]
    lines, offsets, base = [], [], 0
    for plan in plans:
        offsets.append(base)
        for rec in plan.steps:
            rec = dict(rec, step=rec["step"] + base)
            lines.append(json.dumps(rec))
        base += len(plan.steps)
    out = tmp_path / "out"
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    proc = subprocess.run([os.path.join(root, "bin", "trace_run"), "--model", model_folders[name], "--dtype", dtype,
                           "--out", str(out), "--max-tokens", str(max(p.max_tokens for p in plans))],
                          input="\n".join(lines) + "\n", text=True, capture_output=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert proc.stdout.split("\n")[:3] == ["done 0", "done 1", "done 2"]
    assert proc.stdout.count("done ") == base
    for plan, off in zip(plans, offsets):
        outputs = {}
        for step in plan.wanted:
            raw = np.fromfile(out / f"{step + off}.f32", dtype="<f4")
            assert raw.size == len(plan.wanted[step]) * cfg.vocab_size
            outputs[step] = raw
        got = plan.assemble(outputs, {r: len(t) for r, t in reqs.items()}, cfg.vocab_size)
        for rid in reqs:
            helpers.assert_close(got[rid], want[rid], dtype, f"trace_run {dtype} {rid}")


def test_trace_run_reports_a_pool_that_is_too_small(model_folders, tmp_path):
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    rec = {"step": 0, "entries": [{"id": "a", "tokens": list(range(1, 60)), "want": []},
                                  {"id": "b", "tokens": list(range(1, 60)), "want": []}], "end": []}
    proc = subprocess.run([os.path.join(root, "bin", "trace_run"), "--model", model_folders["A"], "--dtype", "float32",
                           "--out", str(tmp_path / "o"), "--max-tokens", "64"],
                          input=json.dumps(rec) + "\n", text=True, capture_output=True, timeout=300)
    assert proc.returncode == 1 and "used up" in proc.stderr and "done 0" not in proc.stdout


def test_trace_run_says_what_is_wrong_with_a_line_or_a_model(model_folders, tmp_path):
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    base = [os.path.join(root, "bin", "trace_run"), "--dtype", "float32", "--out", str(tmp_path / "o"),
            "--max-tokens", "128"]

    def run(model, text):
        return subprocess.run(base + ["--model", model], input=text, text=True, capture_output=True, timeout=300)

    ok = json.dumps({"step": 0, "entries": [{"id": "a", "tokens": [1, 2], "want": [1]}], "end": []}) + "\n"
    cases = {
        "a token id the vocabulary lacks": json.dumps({"step": 1, "entries": [{"id": "a", "tokens": [100000], "want": []}]}),
        "a position past the table": json.dumps({"step": 1, "entries": [{"id": "a", "tokens": [1] * 70, "want": []}]}),
        "not JSON": "{step: 1",
        "want outside the entry": json.dumps({"step": 1, "entries": [{"id": "a", "tokens": [1], "want": [3]}]}),
    }
    for what, line in cases.items():
        proc = run(model_folders["A"], ok + line + "\n")
        assert proc.returncode == 1 and "done 0" in proc.stdout and "done 1" not in proc.stdout, what
        assert "trace_run:" in proc.stderr and "Traceback" not in proc.stderr, (what, proc.stderr)
    proc = run(str(tmp_path / "no_such_model"), ok)
    assert proc.returncode == 1 and "cannot load" in proc.stderr and "Traceback" not in proc.stderr


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_want_may_be_empty_or_partial_and_steps_without_logits_write_no_file(model_folders, dtype):
    cfg = helpers.CONFIGS["A"]
    ids = helpers.random_ids(np.random.default_rng(0), cfg.vocab_size, 40)
    pcfg, w = P.read_model_folder(model_folders["A"])
    want = P.plain_forward(w, pcfg, ids).numpy()
    rep = TraceReplayer(model_folders["A"], dtype, 64, poison=True)
    assert rep.run_step({"step": 0, "entries": [{"id": "x", "tokens": ids[:25], "want": []}], "end": []}) is None
    got = rep.run_step({"step": 1, "entries": [{"id": "x", "tokens": ids[25:], "want": [14, 0]}], "end": ["x"]})
    helpers.assert_close(got, want[[39, 25]], dtype, "partial want")
    with pytest.raises(TraceError, match="outside"):
        rep.run_step({"step": 2, "entries": [{"id": "y", "tokens": [1, 2], "want": [2]}], "end": []})


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_and_first_tokens(model_folders, dtype):
    """One token at a time from the very first token to the last position the model has."""
    cfg = helpers.CONFIGS["B"]
    ids = helpers.random_ids(np.random.default_rng(8), cfg.vocab_size, cfg.block_size)
    pcfg, w = P.read_model_folder(model_folders["B"])
    want = P.plain_forward(w, pcfg, ids).numpy()
    rep = TraceReplayer(model_folders["B"], dtype, cfg.block_size + 8, page_size=8, poison=True)
    rows = [rep.run_step({"step": i, "entries": [{"id": "x", "tokens": [t], "want": [0]}], "end": []}).cpu().numpy()[0]
            for i, t in enumerate(ids)]
    helpers.assert_close(np.stack(rows), want, dtype, "token by token")
    with pytest.raises(ValueError, match="block_size"):       # reference tests/test_cache.py:147-158
        rep.run_step({"step": 999, "entries": [{"id": "x", "tokens": [1], "want": [0]}], "end": []})


@pytest.mark.parametrize("n_req", [17, 40, 64])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_many_requests_decoding_together(model_folders, name, dtype, n_req):
    """Decode steps of 17 to 64 requests (where the products deal the rows out in groups of 16, or
    share the matrix between them): prompts of different lengths enter a few at a time, then all
    requests bring one token a step."""
    cfg = helpers.CONFIGS[name]
    rng = np.random.default_rng(21)
    n_dec = 6
    reqs = {f"r{i}": helpers.random_ids(rng, cfg.vocab_size, int(rng.integers(1, cfg.block_size - n_dec)) + n_dec)
            for i in range(n_req)}
    pcfg, w = P.read_model_folder(model_folders[name])
    want = {rid: P.plain_forward(w, pcfg, ids).numpy() for rid, ids in reqs.items()}
    plan = helpers.TracePlan()
    rids = list(reqs)
    for i in range(0, n_req, 5):       # prompts, five requests a step
        plan.add_step([(r, reqs[r][:-n_dec], len(reqs[r])) for r in rids[i:i + 5]])
    for j in range(n_dec, 0, -1):      # then every request's next token, all in one step
        plan.add_step([(r, reqs[r][len(reqs[r]) - j:len(reqs[r]) - j + 1], len(reqs[r])) for r in rids],
                      end=rids if j == 1 else [])
    replayer = TraceReplayer(model_folders[name], dtype, plan.tight_tokens(16), max_live=n_req, poison=True)
    got = plan.assemble(helpers.run_plan_in_process(replayer, plan), {r: len(t) for r, t in reqs.items()},
                        cfg.vocab_size)
    for rid in reqs:
        helpers.assert_close(got[rid], want[rid], dtype, f"{name} {dtype} {n_req} requests, {rid}")
    assert replayer.cache.check() == 0 and replayer.cache.num_free_pages() == replayer.num_pages


def _far_key_edit(tensors):
    """Makes the last query of the LONG model look mostly at one far key whose value is the
    opposite of its own.  Queries and keys share one enlarged projection that reads the first 40
    channels, values read the last 8 (enlarged too); token 59's embedding is token 60's with the
    last 8 channels negated, which leaves LayerNorm's statistics almost alone.  So 60's query
    scores as high with 59's key as with its own, among hundreds of others, and 59's value
    cancels 60's.  Positions are made faint so that a token looks alike wherever it stands."""
    c, cut = 48, 40
    qkv = tensors["blocks.0.attn.qkv.weight"].float()
    qkv[:c] *= 2.5
    qkv[:c, cut:] = 0
    qkv[c:2 * c] = qkv[:c]
    qkv[2 * c:, :cut] = 0
    qkv[2 * c:] *= 4.0
    tensors["blocks.0.attn.qkv.weight"] = qkv.to(torch.bfloat16)
    bias = tensors["blocks.0.attn.qkv.bias"].float()
    bias[c:2 * c] = bias[:c]
    tensors["blocks.0.attn.qkv.bias"] = bias.to(torch.bfloat16)
    emb = tensors["tok_emb.weight"].float()
    emb[59] = emb[60]
    emb[59, cut:] = -emb[60, cut:]
    tensors["tok_emb.weight"] = emb.to(torch.bfloat16)
    tensors["pos_emb.weight"] = (tensors["pos_emb.weight"].float() * 0.05).to(torch.bfloat16)


@pytest.mark.parametrize("far", [3, 15, 16, 255, 256, 447])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_far_key_among_hundreds_decides_the_result(tmp_path, dtype, far):
    folder = helpers.write_model(str(tmp_path / "long"), "LONG", edit=_far_key_edit)
    cfg = helpers.CONFIGS["LONG"]
    rng = np.random.default_rng(far)
    n = 600
    ids = rng.integers(0, 59, n).tolist()     # tokens 59 and 60 appear only where they are put
    ids[far] = 59
    ids[-1] = 60
    pcfg, w = P.read_model_folder(folder)
    # the construction works: in the plain implementation the last query puts most weight on `far`
    x = P.plain_embed(torch.tensor(ids), w["tok_emb.weight"], w["pos_emb.weight"])
    h = P.plain_layer_norm(x, w["blocks.0.ln1.weight"], w["blocks.0.ln1.bias"], cfg.layer_norm_eps)
    q, k, v = P.plain_split_heads(P.plain_linear(h, w["blocks.0.attn.qkv.weight"], w["blocks.0.attn.qkv.bias"]), 1)
    probs = torch.softmax((q[0, -1] @ k[0].t()) / 48 ** 0.5, -1)
    assert probs[far] > 0.2 and probs[far] > probs[-1], (probs[far].item(), probs[-1].item())
    want = P.plain_forward(w, pcfg, ids).numpy()
    rep = TraceReplayer(folder, dtype, 640, poison=True)
    rep.run_step({"step": 0, "entries": [{"id": "x", "tokens": ids[:-40], "want": []}], "end": []})
    got = rep.run_step({"step": 1, "entries": [{"id": "x", "tokens": ids[-40:-1], "want": list(range(39))}], "end": []})
    helpers.assert_close(got, want[-40:-1], dtype, "portion over a long cache")
    got = rep.run_step({"step": 2, "entries": [{"id": "x", "tokens": ids[-1:], "want": [0]}], "end": ["x"]})
    helpers.assert_close(got, want[-1:], dtype, f"decode with the deciding key at {far}")
    # and the far key really decides: with another token there the logits move a lot
    other = list(ids)
    other[far] = 7
    moved = np.abs(P.plain_forward(w, pcfg, other).numpy()[-1] - want[-1]).max()
    assert moved > 10 * helpers.TOL[dtype] * max(1.0, np.abs(want[-1]).max())


FAMILY = {
    # the reference family's real widths, head counts and odd vocabulary, with few layers to keep it quick
    "small": dict(n_layer=2, n_embd=768, n_head=12, vocab_size=50257, block_size=1024, bias=True),
    "xl": dict(n_layer=1, n_embd=1600, n_head=25, vocab_size=50257, block_size=1024, bias=True),
    "50M": dict(n_layer=2, n_embd=512, n_head=8, vocab_size=50304, block_size=1024, bias=True),
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("shape", ["small", "xl", "50M"])
def test_real_family_sizes(tmp_path, shape, dtype):
    """Widths 512/768/1600, 25 heads, vocabularies 50257 and 50304: a prompt portion, a second
    portion over the cache, and single tokens, against the plain implementation."""
    from mini_gpt_inference_amd import GPTConfig
    from mini_gpt_inference_amd.weights.random_init import write_random_model
    cfg = GPTConfig("gpt2-mini", layer_norm_eps=1e-5, **FAMILY[shape])
    folder = write_random_model(str(tmp_path / shape), cfg, 7, std_scale=2.0)
    rng = np.random.default_rng(1)
    ids = helpers.random_ids(rng, cfg.vocab_size, 90)
    pcfg, w = P.read_model_folder(folder)
    want = P.plain_forward(w, pcfg, ids).numpy()
    rep = TraceReplayer(folder, dtype, 128, poison=True)
    # no wait between the steps, and each result copied on the device: a step must not disturb the
    # inputs of the one before it while the device is still behind
    got = [rep.run_step({"step": 0, "entries": [{"id": "x", "tokens": ids[:70], "want": [0, 33, 69]}], "end": []}).clone(),
           rep.run_step({"step": 1, "entries": [{"id": "x", "tokens": ids[70:87], "want": [0, 16]}], "end": []}).clone()]
    for i in range(87, 90):
        got.append(rep.run_step({"step": i, "entries": [{"id": "x", "tokens": ids[i:i + 1], "want": [0]}], "end": []}).clone())
    helpers.assert_close(torch.cat(got), want[[0, 33, 69, 70, 86, 87, 88, 89]], dtype, f"{shape} {dtype}")


_family_cache = {}


def _family_model(tmp_path_factory, shape):
    """(folder, config, plain config, plain weights) of a family shape, written once per session."""
    if shape not in _family_cache:
        from mini_gpt_inference_amd import GPTConfig
        from mini_gpt_inference_amd.weights.random_init import write_random_model
        cfg = GPTConfig("gpt2-mini", layer_norm_eps=1e-5, **FAMILY[shape])
        folder = write_random_model(str(tmp_path_factory.mktemp("family") / shape), cfg, 7, std_scale=2.0)
        pcfg, w = P.read_model_folder(folder)
        _family_cache[shape] = (folder, cfg, pcfg, w)
    return _family_cache[shape]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("shape", ["small", "xl", "50M"])
def test_real_family_sizes_mixed_with_page_reuse(tmp_path_factory, shape, dtype):
    """The real widths under the mixed schedule: up to four live requests, portions of some beside
    single tokens of others, a NaN-poisoned pool so small that pages are used again."""
    folder, cfg, pcfg, w = _family_model(tmp_path_factory, shape)
    rng = np.random.default_rng(21)
    reqs = {f"r{i}": helpers.random_ids(rng, cfg.vocab_size, n) for i, n in enumerate([50, 37, 64, 20, 45, 33])}
    plan = helpers.plan_mixed(reqs, np.random.default_rng(8), tail=12)
    replayer = TraceReplayer(folder, dtype, plan.tight_tokens(16), poison=True)
    assert sum(-(-len(t) // 16) for t in reqs.values()) > replayer.num_pages, "no page would be used twice"
    got = plan.assemble(helpers.run_plan_in_process(replayer, plan), {r: len(t) for r, t in reqs.items()},
                        cfg.vocab_size)
    for rid, ids in reqs.items():
        helpers.assert_close(got[rid], P.plain_forward(w, pcfg, ids).numpy(), dtype, f"{shape} {dtype} mixed {rid}")
    assert replayer.cache.check() == 0 and replayer.cache.num_free_pages() == replayer.num_pages


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("cut", ["whole", "halves"])
def test_the_benchmarked_prefill_step(tmp_path_factory, dtype, cut):
    """The prefill step that the benchmark times: two prompts of 1,024 tokens at the 50.9M model's
    widths in one step (and the same prompts as two steps of 512 + 512 over the cache), logits at a
    prompt's first, middle and last positions, against the plain implementation (the reference
    compares a prompt's prefill logits with its oracle, tests/test_cache.py:30-49; a portion's queries
    see the cached keys and their own up to themselves, src/minigpt_infer/batch.py:202-227)."""
    folder, cfg, pcfg, w = _family_model(tmp_path_factory, "50M")
    rng = np.random.default_rng(77)
    prompts = [helpers.random_ids(rng, cfg.vocab_size, 1024) for _ in range(2)]
    rep = TraceReplayer(folder, dtype, 2048, poison=True)
    if cut == "whole":
        steps = [([p for p in prompts], [0, 511, 1023])]
    else:
        steps = [([p[:512] for p in prompts], [0, 511]), ([p[512:] for p in prompts], [0, 511])]
    got, positions, base = [], [], 0
    for i, (portions, rows) in enumerate(steps):
        out = rep.run_step({"step": i, "entries": [{"id": f"p{j}", "tokens": t, "want": rows}
                                                   for j, t in enumerate(portions)], "end": []})
        got.append(out.clone().view(2, len(rows), -1))
        positions += [base + r for r in rows]
        base += len(portions[0])
    got = torch.cat(got, dim=1)
    for j, prompt in enumerate(prompts):
        want = P.plain_forward(w, pcfg, prompt, rows=positions)
        helpers.assert_close(got[j], want, dtype, f"prompt {j}, {cut}, positions {positions}")
    assert rep.cache.num_free_pages() == 0, "the pool was meant to be exactly the two prompts"


def test_the_benchmarked_prefill_step_replayed_from_its_graph(tmp_path_factory):
    """The same step six times with other prompts each time, the requests ended in between so that the
    pages come back: the first comings run eagerly and from the recorded plan, the third is captured, the
    later ones are replays of that graph (whose products include the variants that load straight into
    LDS: the second feed-forward product's inner size is 32 steps).  Every coming is compared with the
    plain implementation."""
    folder, cfg, pcfg, w = _family_model(tmp_path_factory, "50M")
    rng = np.random.default_rng(78)
    rep = TraceReplayer(folder, "bfloat16", 2048, poison=True)
    assert rep.runner.graph_steps
    rows = [0, 700, 1023]
    for i in range(6):
        prompts = [helpers.random_ids(rng, cfg.vocab_size, 1024) for _ in range(2)]
        out = rep.run_step({"step": i, "entries": [{"id": f"r{i}p{j}", "tokens": t, "want": rows}
                                                   for j, t in enumerate(prompts)],
                            "end": [f"r{i}p0", f"r{i}p1"]})
        got = out.clone().view(2, len(rows), -1)
        for j, prompt in enumerate(prompts):
            helpers.assert_close(got[j], P.plain_forward(w, pcfg, prompt, rows=rows), "bfloat16", f"coming {i}, prompt {j}")
    assert rep.runner.num_replayed_steps >= 3
    assert rep.cache.check() == 0 and rep.cache.num_free_pages() == rep.num_pages


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("n_req", [8, 17, 40, 64, 100, 128, 200, 256])
@pytest.mark.parametrize("shape", ["small", "xl", "50M"])
def test_real_family_sizes_many_requests_decoding(tmp_path_factory, shape, dtype, n_req):
    """Decode steps of 8 to 256 requests at the real widths, as logits: the decode products
    change kernels with the rows and the matrix's size (rows dealt out in groups, the inner size
    split over workgroups and its sums left pending, the hand-over to the tiled kernel, the fused
    kernels with one, two and four tokens a workgroup).
    The same step comes several times, so the later ones are graph replays."""
    folder, cfg, pcfg, w = _family_model(tmp_path_factory, shape)
    rng = np.random.default_rng(100 + n_req)
    steps = 4
    seqs = [helpers.random_ids(rng, cfg.vocab_size, int(rng.integers(1, 6)) + steps) for _ in range(n_req)]
    want = [P.plain_forward(w, pcfg, s).numpy() for s in seqs]
    rep = TraceReplayer(folder, dtype, n_req * 16, max_live=n_req, poison=True)
    heads = [len(s) - steps for s in seqs]
    rep.run_step({"step": 0, "entries": [{"id": f"r{i}", "tokens": s[:h], "want": []}
                                         for i, (s, h) in enumerate(zip(seqs, heads))], "end": []})
    for j in range(steps):
        got = rep.run_step({"step": 1 + j, "entries": [{"id": f"r{i}", "tokens": [s[h + j]], "want": [0]}
                                                       for i, (s, h) in enumerate(zip(seqs, heads))], "end": []})
        ref = np.stack([wv[h + j] for wv, h in zip(want, heads)])
        helpers.assert_close(got, ref, dtype, f"{shape} {dtype}: decode step {j} of {n_req} requests")
    assert rep.runner.num_replayed_steps >= 1


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_step_shapes_that_repeat_are_replayed_from_a_graph_with_the_same_logits(model_folders, dtype):
    """Single tokens and portions of four, over and over: from the fourth step of a shape on the
    step is a graph replay; every replay is checked against the plain implementation, with eager
    steps of other shapes between them; a larger step in between makes the workspace grow, which
    retires the graphs captured before it."""
    cfg = helpers.CONFIGS["B"]
    rng = np.random.default_rng(5)
    ids = helpers.random_ids(rng, cfg.vocab_size, 120)
    other = helpers.random_ids(rng, cfg.vocab_size, 90)
    pcfg, w = P.read_model_folder(model_folders["B"])
    want, want_other = P.plain_forward(w, pcfg, ids).numpy(), P.plain_forward(w, pcfg, other).numpy()
    rep = TraceReplayer(model_folders["B"], dtype, 256, poison=True)
    assert rep.runner.graph_steps
    fed, step = 0, 0

    def feed(n, rid="x", seq=ids, ref=want, start=None):
        nonlocal step
        s = fed if start is None else start
        got = rep.run_step({"step": step, "entries": [{"id": rid, "tokens": seq[s:s + n], "want": list(range(n))}],
                            "end": []}).cpu()
        step += 1
        helpers.assert_close(got, ref[s:s + n], dtype, f"step {step}: tokens {s}..{s + n}")

    for _ in range(8):                      # shape (1,): recorded, from the plan, captured, then replays
        feed(1); fed += 1
    first = rep.runner.num_replayed_steps
    assert first >= 4 and rep.runner.num_planned_steps >= 1
    for _ in range(6):                      # shape (4,) between them
        feed(4); fed += 4
        feed(1); fed += 1
    assert rep.runner.num_replayed_steps >= first + 8
    feed(60, "y", other, want_other, 0)     # a larger step: buffers grow, the graphs are stale
    before = rep.runner.num_replayed_steps
    for _ in range(8):
        feed(1); fed += 1
        feed(4); fed += 4
    assert rep.runner.num_replayed_steps >= before + 8   # captured again and replayed again
    for i in range(60, 64):                 # and the other request goes on where it stood
        feed(1, "y", other, want_other, i)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_shape_seen_before_is_launched_from_its_recorded_plan(model_folders, dtype):
    """Without HIP graphs every repeat of a step shape makes its launches from the plan recorded at
    the shape's first coming (one call into the kernel library instead of the model's Python); every
    such step is checked against the plain implementation, other shapes come between them, and a
    larger step that makes the workspace grow retires the plans, which are then recorded again."""
    cfg = helpers.CONFIGS["A"]
    rng = np.random.default_rng(8)
    ids = helpers.random_ids(rng, cfg.vocab_size, 60)
    other = helpers.random_ids(rng, cfg.vocab_size, 50)
    pcfg, w = P.read_model_folder(model_folders["A"])
    want, want_other = P.plain_forward(w, pcfg, ids).numpy(), P.plain_forward(w, pcfg, other).numpy()
    rep = TraceReplayer(model_folders["A"], dtype, 128, page_size=4, poison=True)
    rep.runner.graph_steps = False
    assert rep.runner.plan_steps
    fed = step = 0

    def feed(n, rid="x", seq=ids, ref=want, start=None):
        nonlocal step
        s = fed if start is None else start
        got = rep.run_step({"step": step, "entries": [{"id": rid, "tokens": seq[s:s + n], "want": list(range(n))}],
                            "end": []}).cpu()
        step += 1
        helpers.assert_close(got, ref[s:s + n], dtype, f"step {step}: tokens {s}..{s + n}")

    for _ in range(2):                           # both shapes twice: the workspace has all its buffers by then
        feed(3); fed += 3
        feed(1); fed += 1
    settled = rep.runner.num_planned_steps
    for _ in range(3):
        feed(3); fed += 3
        feed(1); fed += 1
    assert rep.runner.num_planned_steps == settled + 6 and rep.runner.num_replayed_steps == 0
    feed(40, "y", other, want_other, 0)          # the workspace grows: the plans hold stale addresses
    before = rep.runner.num_planned_steps
    feed(3); fed += 3
    feed(1); fed += 1
    assert rep.runner.num_planned_steps == before, "a plan recorded before the workspace grew was used"
    feed(3); fed += 3
    feed(1); fed += 1
    before = rep.runner.num_planned_steps
    for _ in range(3):
        feed(3); fed += 3
        feed(1); fed += 1
    assert rep.runner.num_planned_steps == before + 6
    for i in range(40, 44):                      # the other request goes on where it stood, from its own plans
        feed(1, "y", other, want_other, i)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_a_plan_holds_what_the_models_python_launches_whatever_the_contexts(model_folders, name, dtype):
    """A recorded plan is valid for every step of its shape only if no launcher argument comes from the
    host's view of the step beyond the shape (context lengths, the longest sequence).  With
    ModelRunner.verify_plans a step whose shape has a plan goes through the model's Python again and
    its launches are compared with the plan's, argument for argument: shapes with single tokens,
    portions and both, at growing and very different context lengths."""
    cfg = helpers.CONFIGS[name]
    rng = np.random.default_rng(12)
    seqs = {rid: helpers.random_ids(rng, cfg.vocab_size, cfg.block_size) for rid in "abc"}
    pcfg, w = P.read_model_folder(model_folders[name])
    want = {rid: P.plain_forward(w, pcfg, s).numpy() for rid, s in seqs.items()}
    rep = TraceReplayer(model_folders[name], dtype, 3 * cfg.block_size, poison=True)
    rep.runner.graph_steps = False
    rep.runner.verify_plans = True
    fed = {rid: 0 for rid in seqs}

    def run(parts):
        entries = [{"id": rid, "tokens": seqs[rid][fed[rid]:fed[rid] + n], "want": [n - 1]} for rid, n in parts]
        got = rep.run_step({"step": 0, "entries": entries, "end": []}).cpu()
        for row, (rid, n) in enumerate(parts):
            helpers.assert_close(got[row], want[rid][fed[rid] + n - 1], dtype, f"{rid} +{n} at {fed[rid]}")
            fed[rid] += n

    run([("a", 30), ("b", 2)])          # contexts that differ from the start
    run([("c", 1)])
    for _ in range(2):                   # the workspace has all its buffers after the first round
        run([("a", 1), ("b", 1), ("c", 1)])
        run([("a", 1), ("b", 5)])
        run([("c", 7)])
        run([("b", 1)])
    checked = rep.runner.num_planned_steps
    for _ in range(4):
        run([("a", 1), ("b", 1), ("c", 1)])
        run([("a", 1), ("b", 5)])
        run([("c", 7)])
        run([("b", 1)])
    assert rep.runner.num_planned_steps >= checked + 16


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_steps_of_a_bucket_are_replayed_from_one_padded_graph(model_folders, dtype, name):
    """Steps whose shapes never repeat but fall into one bucket of capacities (tokens, requests, logit
    rows, leading single tokens): the third one makes the bucket's padded graph, the later ones are
    replays of it with other requests, other cuts and other numbers of single tokens, each checked
    against the plain implementation; eager steps of another bucket come between them."""
    cfg = helpers.CONFIGS[name]
    rng = np.random.default_rng(9)
    limit = cfg.block_size
    seqs = {rid: helpers.random_ids(rng, cfg.vocab_size, min(limit, n)) for rid, n in
            (("a", 60), ("b", 64), ("c", 58), ("d", 40))}
    pcfg, w = P.read_model_folder(model_folders[name])
    want = {rid: P.plain_forward(w, pcfg, s).numpy() for rid, s in seqs.items()}
    rep = TraceReplayer(model_folders[name], dtype, 512, poison=True)
    assert rep.runner.graph_steps
    fed = {rid: 0 for rid in seqs}
    step = 0

    def run(parts):
        """parts: [(request, tokens to feed)], single tokens first as a scheduler would put them."""
        nonlocal step
        entries = []
        for rid, n in parts:
            s = fed[rid]
            entries.append({"id": rid, "tokens": seqs[rid][s:s + n], "want": [n - 1]})
        got = rep.run_step({"step": step, "entries": entries, "end": []}).cpu()
        for row, (rid, n) in enumerate(parts):
            helpers.assert_close(got[row], want[rid][fed[rid] + n - 1], dtype, f"step {step}: {rid} +{n}")
            fed[rid] += n
        step += 1

    run([("a", 9), ("b", 3)])           # everyone has a context before the single tokens start
    run([("c", 2), ("d", 5)])
    # the bucket: 17..20 tokens, 3..4 requests and logit rows, 1..16 leading single tokens
    plan = [[("a", 1), ("b", 1), ("c", 15), ("d", 2)],
            [("d", 1), ("a", 1), ("b", 16)],
            [("c", 1), ("a", 2), ("b", 14), ("d", 3)],      # third step of the bucket: captured here
            [("b", 1), ("c", 1), ("d", 1), ("a", 14)],
            [("a", 1), ("d", 1), ("c", 17)],
            [("d", 1), ("b", 1), ("a", 1), ("c", 15)],
            [("c", 1), ("a", 17), ("d", 2)]]
    before = rep.runner.num_replayed_steps
    for i, parts in enumerate(plan):
        run(parts)
        if i == 3:
            run([("b", 2)])             # another bucket in between, eagerly
    assert rep.runner.num_replayed_steps >= before + 4

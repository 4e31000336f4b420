"""The parts of a model, each alone and put together in other ways than the one architecture
does: other sizes and constants, key/value groups, a window, an untied head, no positions, a
layer that runs twice, a layer that reads another layer's cache, and a toy mixer with state of
its own that is defined here and registered without touching the framework."""

import math

import numpy as np
import pytest
import torch

import helpers
import plain_gpt as P
from mini_gpt_inference_amd import EngineConfig, SamplingParams
from mini_gpt_inference_amd.cache.kv_store import KVStore
from mini_gpt_inference_amd.cache.manager import CacheManager, GroupGeometry
from mini_gpt_inference_amd.engine.llm_engine import LLMEngine
from mini_gpt_inference_amd.engine.step import ModelRunner
from mini_gpt_inference_amd.ops.linear import LazyNorm, as_tensor
from mini_gpt_inference_amd.parts.base import (CacheBinding, MATRIX, PartSpec, StateNeed, WeightRequest,
                                               register_mixer)
from mini_gpt_inference_amd.parts.mixers import Mixer
from mini_gpt_inference_amd.parts.model import DecoderModel, LayerRun, LayerSpec, ModelSpec

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda")
TDT = {"float32": torch.float32, "bfloat16": torch.bfloat16}


# ----------------------------------------------------------------------------- a toy mixer with state
@register_mixer("toy_decay")
class ToyDecayMixer(Mixer):
    """s_t = decay * s_{t-1} + h_t (s starts at zero with a request's first token); out_t = s_t W^T.
    One float32 vector of state per request, kept in the engine's state slots.  Written with
    library calls: it is a test's part, not the product's."""

    def __init__(self, width: int, decay: float) -> None:
        self.width, self.decay = int(width), float(decay)
        self.mix_weight = None

    def weight_requests(self):
        return {"mix_weight": WeightRequest((self.width, self.width), MATRIX)}

    def cache_need(self):
        return StateNeed(self.width)

    def forward_add(self, ctx, h, x, binding, position):
        assert binding.kind == "state"
        pool = ctx.state_pools[binding.index]
        hn = as_tensor(ctx, h)[:ctx.n_tokens].float()
        w = self.mix_weight.float()
        t = 0
        for slot, ctx_len, q_len in zip(ctx.host_state_slots, ctx.host_ctx_lens, ctx.host_q_lens):
            s = torch.zeros(self.width, device=x.device) if ctx_len == 0 else pool[slot].clone()
            for j in range(q_len):
                s = self.decay * s + hn[t]
                x[t] += s @ w.t()
                t += 1
            pool[slot] = s


def plain_toy(h, w, decay):
    s = torch.zeros(h.shape[1], dtype=P.DT)
    out = []
    for t in range(h.shape[0]):
        s = decay * s + h[t]
        out.append(s @ w.t())
    return torch.stack(out)


# ----------------------------------------------------------------------------- building small models
def _norm(prefix, c, eps, bias=True):
    w = {"weight": prefix + "weight"}
    if bias:
        w["bias"] = prefix + "bias"
    return PartSpec("layer_norm", {"width": c, "eps": eps, "bias": bias}, w)


def _attn_layer(i, c, h, hk, d, window, scale, hidden, eps):
    p = f"L{i}."
    return LayerSpec(
        arrangement=PartSpec("pre_norm", {"width": c}),
        norm1=_norm(p + "n1.", c, eps),
        mixer=PartSpec("paged_causal_attention",
                       {"width": c, "n_head": h, "head_dim": d, "bias": True, "n_kv_head": hk, "scale": scale,
                        "window": window},
                       {"qkv_weight": p + "qkv.w", "qkv_bias": p + "qkv.b", "proj_weight": p + "o.w",
                        "proj_bias": p + "o.b"}),
        norm2=_norm(p + "n2.", c, eps),
        feed_forward=PartSpec("dense_mlp", {"width": c, "hidden": hidden, "bias": True, "activation": "gelu_tanh"},
                              {"fc_weight": p + "fc.w", "fc_bias": p + "fc.b", "proj_weight": p + "pr.w",
                               "proj_bias": p + "pr.b"}))


def _toy_layer(i, c, decay, hidden, eps):
    p = f"L{i}."
    base = _attn_layer(i, c, 1, 1, 16, 0, 1.0, hidden, eps)
    return LayerSpec(base.arrangement, base.norm1,
                     PartSpec("toy_decay", {"width": c, "decay": decay}, {"mix_weight": p + "mix.w"}),
                     base.norm2, base.feed_forward)


def _random_weights(model, seed, scale=0.12):
    """Matrices of standard deviation about 1/sqrt(width): every linear map keeps magnitudes, so
    that five runs deep a bfloat16 rounding is not amplified from layer to layer."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, req in model.weight_requests().items():
        t = torch.randn(req.shape, generator=g) * (scale if len(req.shape) == 2 else 0.1)
        if name.endswith("n1.weight") or name.endswith("n2.weight") or name.endswith("nf.weight"):
            t = 1 + t
        out[name] = t.to(torch.bfloat16)      # values that both dtypes hold exactly
    return out


def _bind(model, weights, dtype):
    tensors = {}
    for name, req in model.weight_requests().items():
        t = weights[name]
        tensors[name] = t.to(torch.float32 if (req.role == "vector" or dtype == "float32") else torch.bfloat16).to(DEV)
    model.bind(tensors)


def _runner(model, dtype, page_size=4, num_pages=64, max_requests=4, poison=True):
    geo = [GroupGeometry(page_size, num_pages, g.window) for g in model.cache_layout.groups]
    cache = CacheManager(geo, max_requests)
    store = KVStore(model.cache_layout, geo, max_requests, TDT[dtype], DEV, poison=poison)
    return ModelRunner(model, cache, store, TDT[dtype], DEV, model.spec.max_positions), cache


# the plain counterparts of the parts, from the functions of plain_gpt
def _pl_norm(x, w, prefix, eps):
    return P.plain_layer_norm(x, w[prefix + "weight"].double(), w[prefix + "bias"].double(), eps)


def _pl_attn(h, w, p, n_head, hk, scale, window, kv_from=None):
    qkv = P.plain_linear(h, w[p + "qkv.w"].double(), w[p + "qkv.b"].double())
    q, k, v = P.plain_split_heads(qkv, n_head, hk)
    if kv_from is not None:
        k, v = kv_from
    y = P.plain_causal_attention(q, k, v, scale=scale, window=window)
    return P.plain_linear(y, w[p + "o.w"].double(), w[p + "o.b"].double()), (k, v)


def _pl_mlp(h, w, p):
    u = P.plain_gelu_tanh(P.plain_linear(h, w[p + "fc.w"].double(), w[p + "fc.b"].double()))
    return P.plain_linear(u, w[p + "pr.w"].double(), w[p + "pr.b"].double())


# ----------------------------------------------------------------------------- the model under test
C, H, HK, D, HID, EPS, V, WINDOW, SCALE = 96, 6, 2, 16, 80, 3e-4, 91, 7, 0.31


def _spec(order, positions="learned_absolute", tied=False):
    layers = (_attn_layer(0, C, H, HK, D, WINDOW, SCALE, HID, EPS),      # grouped heads, a window, its own scale
              _toy_layer(1, C, 0.5, HID, EPS),                            # state instead of keys and values
              _attn_layer(2, C, H, H, D, 0, 1 / math.sqrt(D), HID, EPS))  # all keys: another cache group
    pos = (PartSpec("learned_absolute", {"max_positions": 50, "width": C}, {"weight": "pos.w"})
           if positions == "learned_absolute" else PartSpec("none"))
    return ModelSpec(width=C, vocab_size=V,
                     embedding=PartSpec("token_embedding", {"vocab_size": V, "width": C}, {"weight": "emb.w"}),
                     position=pos, layers=layers, order=tuple(order), final_norm=_norm("nf.", C, EPS),
                     head=PartSpec("linear_head", {"vocab_size": V, "width": C, "tied": tied},
                                   {"weight": "emb.w" if tied else "head.w"}),
                     max_positions=50 if positions == "learned_absolute" else None)


ORDER = (LayerRun(0), LayerRun(1), LayerRun(2), LayerRun(0), LayerRun(2, reads_cache_of=2))


def _plain_model(w, ids, order=ORDER, positions=True, tied=False):
    x = P.plain_embed(torch.tensor(ids), w["emb.w"].double(), w["pos.w"].double() if positions else None)
    caches = {}
    for i, run in enumerate(order):
        p = f"L{run.layer}."
        h = _pl_norm(x, w, p + "n1.", EPS)
        if run.layer == 1:
            x = x + plain_toy(h, w[p + "mix.w"].double(), 0.5)
        else:
            hk, window, scale = (HK, WINDOW, SCALE) if run.layer == 0 else (H, 0, 1 / math.sqrt(D))
            kv = caches[run.reads_cache_of] if run.reads_cache_of is not None else None
            a, caches[i] = _pl_attn(h, w, p, H, hk, scale, window, kv_from=kv)
            x = x + a
        x = x + _pl_mlp(_pl_norm(x, w, p + "n2.", EPS), w, p)
    return _pl_norm(x, w, "nf.", EPS) @ w["emb.w" if tied else "head.w"].double().t()


def test_cache_layout_groups_runs_by_what_their_mixers_keep():
    layout = DecoderModel(_spec(ORDER)).cache_layout
    assert [(g.n_kv_head, g.window, g.n_pools) for g in layout.groups] == [(HK, WINDOW, 2), (H, 0, 1)]
    assert layout.state_numels == [C]
    assert all(sorted(b) == ["mixer"] for b in layout.run_bindings)       # one mixer a layer: one binding a run
    kinds = [(b.kind, b.group, b.index, b.writes) for b in layout.bindings]
    assert kinds == [("kv", 0, 0, True), ("state", -1, 0, True), ("kv", 1, 0, True), ("kv", 0, 1, True),
                     ("kv", 1, 0, False)]
    with pytest.raises(ValueError, match="earlier run"):
        DecoderModel(_spec((LayerRun(0, reads_cache_of=0),)))
    with pytest.raises(ValueError, match="different needs"):
        DecoderModel(_spec((LayerRun(0), LayerRun(2, reads_cache_of=0))))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("variant", ["full", "no-positions-tied-head"])
def test_mixed_layers_repeated_layer_shared_cache_and_toy_state(dtype, variant):
    positions, tied = variant == "full", variant != "full"
    model = DecoderModel(_spec(ORDER, "learned_absolute" if positions else "none", tied))
    weights = _random_weights(model, 5)
    _bind(model, weights, dtype)
    rng = np.random.default_rng(1)
    reqs = [rng.integers(0, V, n).tolist() for n in (23, 9, 40)]
    want = [_plain_model(weights, ids, positions=positions, tied=tied).numpy() for ids in reqs]

    # whole, then in portions beside single tokens of the others, with pages of the window group returning
    runner, cache = _runner(model, dtype)
    slots = [cache.acquire_slot() for _ in reqs]
    for s, ids in zip(slots, reqs):
        assert cache.reserve(s, len(ids))
    whole = runner.step(slots, [0] * 3, [len(r) for r in reqs], sum(reqs, []), list(range(sum(map(len, reqs)))))
    off = 0
    for ids, w_ in zip(reqs, want):
        helpers.assert_close(whole[off:off + len(ids)], w_, dtype, f"whole {variant}")
        off += len(ids)
    for s in slots:
        cache.free_slot(s)

    slots = [cache.acquire_slot() for _ in reqs]
    done = [0, 0, 0]
    got = [[] for _ in reqs]
    sizes = [[5, 1, 1, 7, 2, 1, 6], [2, 3, 1, 1, 2], [16, 1, 9, 1, 1, 12]]
    step = 0
    while any(d < len(r) for d, r in zip(done, reqs)):
        batch = []
        for i, ids in enumerate(reqs):
            if done[i] < len(ids) and (step + i) % 4 != 3:        # now and then a request sits a step out
                q = min(sizes[i][step % len(sizes[i])], len(ids) - done[i])
                batch.append((i, q))
        step += 1
        if not batch:
            continue
        for i, q in batch:
            assert cache.reserve(slots[i], done[i] + q)
        toks = sum((reqs[i][done[i]:done[i] + q] for i, q in batch), [])
        out = runner.step([slots[i] for i, _ in batch], [done[i] for i, _ in batch], [q for _, q in batch], toks,
                          list(range(len(toks))))
        o = 0
        for i, q in batch:
            got[i].append(out[o:o + q].cpu())
            o += q
            done[i] += q
            cache.release_passed(slots[i], done[i])
    for i in range(3):
        helpers.assert_close(torch.cat(got[i]), want[i], dtype, f"cut {variant} request {i}")
    # the window group gave pages back while the request was still running
    assert cache.held_pages(slots[2], 0) < cache.pages_needed(40, 0) == cache.held_pages(slots[2], 1)
    assert cache.check() == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_each_part_alone(dtype):
    """Norm, feed-forward, mixer, embedding with and without positions, head: called directly."""
    model = DecoderModel(_spec((LayerRun(0),)))
    weights = _random_weights(model, 9)
    _bind(model, weights, dtype)
    runner, cache = _runner(model, dtype)
    tdt = TDT[dtype]
    ids = np.random.default_rng(2).integers(0, V, 20).tolist()
    slot = cache.acquire_slot()
    cache.reserve(slot, 20)
    w64 = {k: v.double() for k, v in weights.items()}

    def ctx_for(start, q):
        arena = runner.arena(q, 1, q)
        shape = runner.describe(arena, [slot], [start], [q], ids[start:start + q], list(range(q)))
        arena.upload()
        return runner.context(arena, shape, padded=False)

    ctx = ctx_for(0, 13)
    layer = model.layers[0]
    g = torch.Generator().manual_seed(0)
    x0 = torch.randn(13, C, generator=g)

    # embedding, with the learned positions and with none
    x = torch.empty(13, C, device=DEV)
    model.embedding.forward(ctx, model.position, x)
    helpers.assert_close(x, P.plain_embed(torch.tensor(ids[:13]), w64["emb.w"], w64["pos.w"]), "float32", "embed+pos")
    from mini_gpt_inference_amd.parts.positions import NoPositions
    model.embedding.forward(ctx, NoPositions(), x)
    helpers.assert_close(x, P.plain_embed(torch.tensor(ids[:13]), w64["emb.w"], None), "float32", "embed")

    # norm
    out = torch.empty(13, C, dtype=tdt, device=DEV)
    layer.norm1.forward(ctx, x0.to(DEV), out, 13)
    helpers.assert_close(out, _pl_norm(x0.double(), w64, "L0.n1.", EPS), dtype, "norm")

    # feed-forward: adds into the residual stream, from an uncomputed norm and from a tensor
    for lazy in (True, False):
        xr = x0.clone().to(DEV)
        h = LazyNorm(layer.norm2, xr, 13) if lazy else out
        layer.feed_forward.forward_add(ctx, h, xr)
        hn = _pl_norm(x0.double(), w64, "L0.n2." if lazy else "L0.n1.", EPS)
        helpers.assert_close(xr, x0.double() + _pl_mlp(hn, w64, "L0."), dtype, f"feed-forward lazy={lazy}")

    # mixer: a portion of 13, then 7 more one by one, against the whole sequence at once
    x_all = torch.randn(20, C, generator=g)
    h_all = _pl_norm(x_all.double(), w64, "L0.n1.", EPS)
    want = x_all.double() + _pl_attn(h_all, w64, "L0.", H, HK, SCALE, WINDOW)[0]
    binding = model.cache_layout.bindings[0]
    xr = x_all[:13].clone().to(DEV)
    layer.mixer.forward_add(ctx, LazyNorm(layer.norm1, xr, 13), xr, binding, model.position)
    helpers.assert_close(xr, want[:13], dtype, "mixer portion")
    for t in range(13, 20):
        c1 = ctx_for(t, 1)
        xr = x_all[t:t + 1].clone().to(DEV)
        layer.mixer.forward_add(c1, LazyNorm(layer.norm1, xr, 1), xr, binding, model.position)
        helpers.assert_close(xr, want[t:t + 1], dtype, f"mixer decode {t}")

    # head (untied here), float32 logits
    logits = torch.empty(13, V, device=DEV)
    model.head.forward(ctx, out, logits, 13)
    helpers.assert_close(logits, _pl_norm(x0.double(), w64, "L0.n1.", EPS) @ w64["head.w"].t(), dtype, "head")
    assert model.head.weight.data_ptr() != model.embedding.weight.data_ptr()


def test_part_constructors_refuse_what_the_kernels_cannot_do():
    from mini_gpt_inference_amd.parts.base import FEED_FORWARDS, MIXERS
    with pytest.raises(ValueError, match="up to 256"):
        MIXERS.build(PartSpec("paged_causal_attention", {"width": 544, "n_head": 2, "head_dim": 272, "bias": False}))
    MIXERS.build(PartSpec("paged_causal_attention", {"width": 40, "n_head": 2, "head_dim": 20, "bias": False}))
    with pytest.raises(ValueError, match="multiple of n_kv_head"):
        MIXERS.build(PartSpec("paged_causal_attention", {"width": 96, "n_head": 6, "head_dim": 16, "bias": False,
                                                         "n_kv_head": 4}))
    with pytest.raises(ValueError, match="no kernel epilogue"):
        FEED_FORWARDS.build(PartSpec("dense_mlp", {"width": 32, "hidden": 64, "bias": False, "activation": "relu"}))
    with pytest.raises(KeyError, match="no mixer of kind"):
        MIXERS.build(PartSpec("nonexistent"))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_model_generates_through_the_engine(dtype):
    """The engine, scheduler and state slots work for a model that no registered architecture describes;
    eviction resets the toy's state because it starts over.  The toy mixer does not declare itself
    graph_safe (it reads host-side lists), so the engine, asked for graphs, still runs every step eagerly."""
    model = DecoderModel(_spec(ORDER))
    weights = _random_weights(model, 12, scale=0.2)
    _bind(model, weights, dtype)
    prompts = [np.random.default_rng(3).integers(0, V, n).tolist() for n in (6, 11, 3)]
    sp = SamplingParams(max_tokens=8, temperature=0.0)
    assert not model.graph_safe
    engine = LLMEngine(model, None, EngineConfig(block_size=4, num_blocks=40, max_batch_size=3, dtype=dtype,
                                                 prefill_chunk=4, use_graph=True))
    got = engine.generate(prompts, sp)
    assert engine.stats()["graph_steps"] == 0 and engine.stats()["replayed_eager_steps"] == 0
    tight = LLMEngine(model, None, EngineConfig(block_size=4, num_blocks=9, max_batch_size=3, dtype=dtype,
                                                use_graph=True))
    got_tight = tight.generate(prompts, sp)
    assert tight.stats()["num_preemptions"] > 0
    for prompt, tokens, tokens_tight in zip(prompts, got, got_tight):
        ids = list(prompt)
        for k, tok in enumerate(tokens):
            logits = _plain_model(weights, ids)[-1].numpy()
            margin = 2 * helpers.TOL[dtype] * max(1.0, np.abs(logits).max())
            assert logits[tok] >= logits.max() - margin
            ids.append(tok)
        if dtype == "float32":
            assert tokens_tight == tokens
    assert engine.cache.check() == 0 and engine.cache.num_free_pages(0) == 40 and engine.cache.num_free_pages(1) == 40


# ----------------------------------------------------------------------------- two more toy parts
# A position encoding that acts on queries and keys, and a feed-forward that routes each token to
# one of several experts: defined and registered here, written with library calls, never part of
# the product.  They show that the hooks of the parts carry such things without a change to the
# framework's files.
from mini_gpt_inference_amd.parts.base import register_feed_forward, register_position  # noqa: E402
from mini_gpt_inference_amd.parts.feedforward import FeedForward  # noqa: E402
from mini_gpt_inference_amd.parts.positions import PositionEncoding  # noqa: E402


@register_position("toy_pair_rotation")
class ToyPairRotation(PositionEncoding):
    """Turns the pair (2i, 2i+1) of every head of q and k by the angle pos * base^(-i / (D/2)), so that
    q.k depends on the distance of the two positions only.  Everything it does is a device operation on
    device tensors, so it declares itself safe for graphs."""

    rotates = True
    graph_safe = True

    def __init__(self, head_dim: int, base: float) -> None:
        self.head_dim, self.base = int(head_dim), float(base)
        self._freq = None

    def rotate(self, ctx, q, k, n_tokens):
        half = self.head_dim // 2
        if self._freq is None:
            self._freq = (self.base ** (-torch.arange(half, dtype=torch.float64) / half)).float().to(q.device)
        ang = ctx.positions[:n_tokens].float()[:, None] * self._freq[None, :]
        cos, sin = ang.cos()[:, None, :], ang.sin()[:, None, :]
        for t in (q, k):
            pairs = t[:n_tokens].float().reshape(n_tokens, -1, half, 2)
            a, b = pairs[..., 0], pairs[..., 1]
            turned = torch.stack((a * cos - b * sin, a * sin + b * cos), dim=-1)
            t[:n_tokens].copy_(turned.reshape(n_tokens, -1))


def plain_pair_rotation(x, positions, base):
    """x: [heads, T, D] float64; positions: [T]."""
    half = x.shape[-1] // 2
    freq = base ** (-torch.arange(half, dtype=P.DT) / half)
    ang = positions.to(P.DT)[:, None] * freq[None, :]
    out = torch.empty_like(x)
    out[..., 0::2] = x[..., 0::2] * ang.cos() - x[..., 1::2] * ang.sin()
    out[..., 1::2] = x[..., 0::2] * ang.sin() + x[..., 1::2] * ang.cos()
    return out


@register_feed_forward("toy_top1_experts")
class ToyTop1Experts(FeedForward):
    """r = h Wr^T; e = argmax r; out = softmax(r)[e] * gelu(h Wfc[e]^T) Wproj[e]^T.  Asks the host which rows
    each expert gets, so it is not safe for graphs and does not say it is."""

    def __init__(self, width: int, hidden: int, n_experts: int) -> None:
        self.width, self.hidden, self.n_experts = int(width), int(hidden), int(n_experts)
        self.router_weight = self.fc_weight = self.proj_weight = None

    def weight_requests(self):
        return {"router_weight": WeightRequest((self.n_experts, self.width), MATRIX),
                "fc_weight": WeightRequest((self.n_experts * self.hidden, self.width), MATRIX),
                "proj_weight": WeightRequest((self.n_experts * self.width, self.hidden), MATRIX)}

    def forward_add(self, ctx, h, x):
        n = ctx.n_tokens
        hn = as_tensor(ctx, h)[:n].float()
        prob = torch.softmax(hn @ self.router_weight.float().t(), dim=-1)
        gate, expert = prob.max(dim=-1)
        fc = self.fc_weight.float().view(self.n_experts, self.hidden, self.width)
        proj = self.proj_weight.float().view(self.n_experts, self.width, self.hidden)
        for e in range(self.n_experts):
            rows = (expert == e).nonzero().flatten()
            if rows.numel():
                u = torch.nn.functional.gelu(hn[rows] @ fc[e].t(), approximate="tanh")
                x[rows] += gate[rows, None] * (u @ proj[e].t())


def plain_top1_experts(h, router, fc, proj, n_experts):
    """Returns the output and the smallest gap between a token's two largest router logits: where
    that gap is within rounding, the choice of expert is not a fact to compare."""
    r = h @ router.t()
    top2 = r.topk(2, dim=-1).values
    prob = torch.softmax(r, dim=-1)
    out = torch.zeros_like(h)
    hidden = fc.shape[0] // n_experts
    for t in range(h.shape[0]):
        e = int(r[t].argmax())
        u = P.plain_gelu_tanh(h[t] @ fc[e * hidden:(e + 1) * hidden].t())
        out[t] = prob[t, e] * (u @ proj[e * h.shape[1]:(e + 1) * h.shape[1]].t())
    return out, float((top2[:, 0] - top2[:, 1]).min())


ROT_BASE, N_EXPERTS, EXPERT_HIDDEN = 40.0, 3, 56


def _rot_spec(order, routed):
    first = _attn_layer(0, C, H, HK, D, WINDOW, SCALE, HID, EPS)
    if routed:
        first = LayerSpec(first.arrangement, first.norm1, first.mixer, first.norm2,
                          PartSpec("toy_top1_experts", {"width": C, "hidden": EXPERT_HIDDEN, "n_experts": N_EXPERTS},
                                   {"router_weight": "L0.router.w", "fc_weight": "L0.experts.fc",
                                    "proj_weight": "L0.experts.pr"}))
    layers = (first, _attn_layer(1, C, H, H, D, 0, 1 / math.sqrt(D), HID, EPS))
    return ModelSpec(width=C, vocab_size=V,
                     embedding=PartSpec("token_embedding", {"vocab_size": V, "width": C}, {"weight": "emb.w"}),
                     position=PartSpec("toy_pair_rotation", {"head_dim": D, "base": ROT_BASE}),
                     layers=layers, order=tuple(order), final_norm=_norm("nf.", C, EPS),
                     head=PartSpec("linear_head", {"vocab_size": V, "width": C, "tied": True}, {"weight": "emb.w"}),
                     max_positions=None)


ROT_ORDER = (LayerRun(0), LayerRun(1), LayerRun(0))


def _plain_rot_model(w, ids, routed, first_position=0):
    """Returns the logits and the smallest router gap met on the way."""
    x = P.plain_embed(torch.tensor(ids), w["emb.w"].double(), None)
    positions = torch.arange(first_position, first_position + len(ids))
    gap = float("inf")
    for run in ROT_ORDER:
        p = f"L{run.layer}."
        hk, window, scale = (HK, WINDOW, SCALE) if run.layer == 0 else (H, 0, 1 / math.sqrt(D))
        h = _pl_norm(x, w, p + "n1.", EPS)
        q, k, v = P.plain_split_heads(P.plain_linear(h, w[p + "qkv.w"].double(), w[p + "qkv.b"].double()), H, hk)
        q, k = plain_pair_rotation(q, positions, ROT_BASE), plain_pair_rotation(k, positions, ROT_BASE)
        y = P.plain_causal_attention(q, k, v, scale=scale, window=window)
        x = x + P.plain_linear(y, w[p + "o.w"].double(), w[p + "o.b"].double())
        h = _pl_norm(x, w, p + "n2.", EPS)
        if routed and run.layer == 0:
            m, g = plain_top1_experts(h, w["L0.router.w"].double(), w["L0.experts.fc"].double(),
                                      w["L0.experts.pr"].double(), N_EXPERTS)
            gap = min(gap, g)
            x = x + m
        else:
            x = x + _pl_mlp(h, w, p)
    return _pl_norm(x, w, "nf.", EPS) @ w["emb.w"].double().t(), gap


def test_plain_pair_rotation_counts_distances_only():
    """What pins the plain rotation: position 0 changes nothing, lengths are kept, the scores q.k depend
    on the distance alone (so a shift of all positions changes no logit), and a wrong sign in one of the
    two lines would break that."""
    g = torch.Generator().manual_seed(4)
    q, k = torch.randn(2, 9, D, generator=g, dtype=P.DT), torch.randn(2, 9, D, generator=g, dtype=P.DT)
    pos = torch.arange(9)
    assert torch.equal(plain_pair_rotation(q[:, :1], pos[:1], ROT_BASE), q[:, :1])
    assert torch.allclose(plain_pair_rotation(q, pos, ROT_BASE).norm(dim=-1), q.norm(dim=-1), rtol=1e-12)
    s0 = plain_pair_rotation(q, pos, ROT_BASE) @ plain_pair_rotation(k, pos, ROT_BASE).transpose(1, 2)
    s7 = plain_pair_rotation(q, pos + 7, ROT_BASE) @ plain_pair_rotation(k, pos + 7, ROT_BASE).transpose(1, 2)
    assert torch.allclose(s0, s7, atol=1e-12)
    assert not torch.allclose(s0, q @ k.transpose(1, 2), atol=1e-3)
    model = DecoderModel(_rot_spec(ROT_ORDER, routed=True))
    w = _random_weights(model, 21)
    ids = np.random.default_rng(8).integers(0, V, 17).tolist()
    a, b = _plain_rot_model(w, ids, True)[0], _plain_rot_model(w, ids, True, first_position=11)[0]
    assert torch.allclose(a, b, atol=1e-10)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("routed", [False, True])
def test_toy_rotation_and_toy_experts_whole_and_cut(dtype, routed):
    model = DecoderModel(_rot_spec(ROT_ORDER, routed))
    assert model.graph_safe == (not routed)
    weights = _random_weights(model, 48)      # a seed with which no token's two best experts come close
    if routed:
        weights["L0.router.w"] = (weights["L0.router.w"] * 4).to(torch.bfloat16)
    _bind(model, weights, dtype)
    rng = np.random.default_rng(6)
    reqs = [rng.integers(0, V, n).tolist() for n in (29, 12)]
    plain = [_plain_rot_model(weights, ids, routed) for ids in reqs]
    want = [p[0].numpy() for p in plain]
    if routed:      # the inputs are only valid if no token's choice of expert hangs on rounding
        assert min(p[1] for p in plain) > 0.25, min(p[1] for p in plain)

    runner, cache = _runner(model, dtype)
    slots = [cache.acquire_slot() for _ in reqs]
    for s, ids in zip(slots, reqs):
        assert cache.reserve(s, len(ids))
    whole = runner.step(slots, [0, 0], [len(r) for r in reqs], sum(reqs, []), list(range(sum(map(len, reqs)))))
    helpers.assert_close(whole[:29], want[0], dtype, "whole 0")
    helpers.assert_close(whole[29:], want[1], dtype, "whole 1")
    for s in slots:
        cache.free_slot(s)

    slots = [cache.acquire_slot() for _ in reqs]
    done, got = [0, 0], [[], []]
    sizes = [[6, 1, 1, 9, 2, 1], [3, 1, 2, 1, 1]]
    step = 0
    while any(d < len(r) for d, r in zip(done, reqs)):
        batch = [(i, min(sizes[i][step % len(sizes[i])], len(reqs[i]) - done[i])) for i in range(2)
                 if done[i] < len(reqs[i])]
        step += 1
        for i, q in batch:
            assert cache.reserve(slots[i], done[i] + q)
        toks = sum((reqs[i][done[i]:done[i] + q] for i, q in batch), [])
        out = runner.step([slots[i] for i, _ in batch], [done[i] for i, _ in batch], [q for _, q in batch], toks,
                          list(range(len(toks))))
        o = 0
        for i, q in batch:
            got[i].append(out[o:o + q].cpu())
            o += q
            done[i] += q
            cache.release_passed(slots[i], done[i])
    for i in range(2):
        helpers.assert_close(torch.cat(got[i]), want[i], dtype, f"cut request {i}")
    assert cache.check() == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_rotation_decodes_from_graphs(dtype):
    """A toy part that says it is safe for graphs is captured with the rest: greedy generation through
    the engine, decode steps replayed from graphs, each token the plain model's choice."""
    model = DecoderModel(_rot_spec(ROT_ORDER, routed=False))
    weights = _random_weights(model, 23, scale=0.2)
    _bind(model, weights, dtype)
    prompts = [np.random.default_rng(5).integers(0, V, n).tolist() for n in (7, 4)]
    engine = LLMEngine(model, None, EngineConfig(block_size=4, num_blocks=40, max_batch_size=2, dtype=dtype,
                                                 use_graph=True))
    got = engine.generate(prompts, SamplingParams(max_tokens=12, temperature=0.0))
    assert engine.stats()["graph_steps"] > 0
    for prompt, tokens in zip(prompts, got):
        ids = list(prompt)
        for tok in tokens:
            logits = _plain_rot_model(weights, ids, False)[0][-1].numpy()
            margin = 2 * helpers.TOL[dtype] * max(1.0, np.abs(logits).max())
            assert logits[tok] >= logits.max() - margin
            ids.append(tok)


# ----------------------------------------------------------------------------- a toy arrangement
from mini_gpt_inference_amd.parts.base import register_arrangement      # noqa: E402
from mini_gpt_inference_amd.parts.block import Arrangement              # noqa: E402


@register_arrangement("toy_parallel")
class ToyParallel(Arrangement):
    """x = x + attention(h) + state_mixer(h) + ff(h) with h = norm(x): one norm, and two mixers beside
    the feed-forward, all reading the same normed rows.  Defined here and registered without a change
    to the framework: a layer is a map of roles to parts, and this arrangement names other roles than
    the pre-norm block does."""

    roles = ("norm", "attention", "memory", "feed_forward")

    def __init__(self, width: int) -> None:
        self.width = int(width)

    def run(self, ctx, x, parts, bindings, position) -> None:
        h = as_tensor(ctx, LazyNorm(parts["norm"], x, ctx.n_rows)).clone()      # every branch reads the rows as they were
        parts["attention"].forward_add(ctx, h, x, bindings["attention"], position)
        parts["memory"].forward_add(ctx, h, x, bindings["memory"], position)
        parts["feed_forward"].forward_add(ctx, h, x)


def _parallel_spec():
    a0, a1 = (_attn_layer(i, C, H, H, D, 0, 1 / math.sqrt(D), HID, EPS) for i in (0, 1))
    parallel = LayerSpec(PartSpec("toy_parallel", {"width": C}),
                         parts={"norm": ("norm", a1.norm1), "attention": ("mixer", a1.mixer),
                                "memory": ("mixer", PartSpec("toy_decay", {"width": C, "decay": 0.25},
                                                             {"mix_weight": "L1.mix.w"})),
                                "feed_forward": ("feed_forward", a1.feed_forward)})
    return ModelSpec(width=C, vocab_size=V,
                     embedding=PartSpec("token_embedding", {"vocab_size": V, "width": C}, {"weight": "emb.w"}),
                     position=PartSpec("learned_absolute", {"max_positions": 50, "width": C}, {"weight": "pos.w"}),
                     layers=(a0, parallel), order=(LayerRun(0), LayerRun(1), LayerRun(0), LayerRun(1)),
                     final_norm=_norm("nf.", C, EPS),
                     head=PartSpec("linear_head", {"vocab_size": V, "width": C, "tied": True}, {"weight": "emb.w"}),
                     max_positions=50)


def _plain_parallel_model(w, ids):
    x = P.plain_embed(torch.tensor(ids), w["emb.w"].double(), w["pos.w"].double())
    for layer in (0, 1, 0, 1):
        p = f"L{layer}."
        h = _pl_norm(x, w, p + "n1.", EPS)
        a, _ = _pl_attn(h, w, p, H, H, 1 / math.sqrt(D), 0)
        if layer == 0:
            x = x + a
            x = x + _pl_mlp(_pl_norm(x, w, p + "n2.", EPS), w, p)
        else:
            x = x + a + plain_toy(h, w[p + "mix.w"].double(), 0.25) + _pl_mlp(h, w, p)
    return _pl_norm(x, w, "nf.", EPS) @ w["emb.w"].double().t()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_toy_arrangement_with_one_norm_and_two_mixers(dtype):
    """A parallel block registered by the test: its layer has the roles norm / attention / memory /
    feed_forward, the model gives each of its two mixers a cache of its own in every run (pages for
    one, a state slot for the other), and steps cut anywhere give the plain model's logits."""
    model = DecoderModel(_parallel_spec())
    layout = model.cache_layout
    assert [sorted(b) for b in layout.run_bindings] == [["mixer"], ["attention", "memory"]] * 2
    assert [g.n_pools for g in layout.groups] == [4] and layout.state_numels == [C, C]
    assert [layout.run_bindings[i]["memory"].index for i in (1, 3)] == [0, 1]
    assert not model.graph_safe                              # the toy parts make no such promise
    with pytest.raises(ValueError, match="arranges the parts"):
        DecoderModel(ModelSpec(**{**_parallel_spec().__dict__, "layers": (
            LayerSpec(PartSpec("toy_parallel", {"width": C}), norm1=_norm("L0.n1.", C, EPS)),)}))
    weights = _random_weights(model, 21)
    _bind(model, weights, dtype)
    rng = np.random.default_rng(4)
    reqs = [rng.integers(0, V, n).tolist() for n in (19, 33)]
    want = [_plain_parallel_model(weights, ids).numpy() for ids in reqs]
    runner, cache = _runner(model, dtype)
    slots = [cache.acquire_slot() for _ in reqs]
    done = [0, 0]
    got = [[], []]
    sizes = [[6, 1, 1, 4, 1, 2, 9], [11, 1, 7, 1, 1, 20]]
    step = 0
    while any(d < len(r) for d, r in zip(done, reqs)):
        batch = [(i, min(sizes[i][step % len(sizes[i])], len(reqs[i]) - done[i])) for i in range(2)
                 if done[i] < len(reqs[i])]
        step += 1
        for i, q in batch:
            assert cache.reserve(slots[i], done[i] + q)
        toks = sum((reqs[i][done[i]:done[i] + q] for i, q in batch), [])
        out = runner.step([slots[i] for i, _ in batch], [done[i] for i, _ in batch], [q for _, q in batch], toks,
                          list(range(len(toks))))
        o = 0
        for i, q in batch:
            got[i].append(out[o:o + q].cpu())
            o += q
            done[i] += q
    for i in range(2):
        helpers.assert_close(torch.cat(got[i]), want[i], dtype, f"parallel block, request {i}")


# ----------------------------------------------------------------------------- two parts of one kind in a row
@register_arrangement("toy_twice")
class ToyTwice(Arrangement):
    """x += attention_a(norm_a(x)); x += attention_b(norm_b(x)); x += ff_a(norm_c(x)); x += ff_b(norm_d(x)):
    two mixers of one kind and two feed-forwards of one kind follow each other, each reading the
    residual as the one before left it (in a decode step of few rows: as sums still pending)."""

    takes_pending_residual = True
    graph_safe = True
    plan_safe = True
    roles = ("norm_a", "attention_a", "norm_b", "attention_b", "norm_c", "ff_a", "norm_d", "ff_b")

    def __init__(self, width: int) -> None:
        self.width = int(width)

    def run(self, ctx, x, parts, bindings, position) -> None:
        n = ctx.n_rows
        for norm, mixer in (("norm_a", "attention_a"), ("norm_b", "attention_b")):
            parts[mixer].forward_add(ctx, LazyNorm(parts[norm], x, n), x, bindings[mixer], position)
        for norm, ff in (("norm_c", "ff_a"), ("norm_d", "ff_b")):
            parts[ff].forward_add(ctx, LazyNorm(parts[norm], x, n), x)


TW_C, TW_H, TW_D, TW_HID = 128, 4, 32, 192


def _twice_spec():
    a, b = (_attn_layer(i, TW_C, TW_H, TW_H, TW_D, 0, 1 / math.sqrt(TW_D), TW_HID, EPS) for i in (0, 1))
    layer = LayerSpec(PartSpec("toy_twice", {"width": TW_C}),
                      parts={"norm_a": ("norm", a.norm1), "attention_a": ("mixer", a.mixer),
                             "norm_b": ("norm", b.norm1), "attention_b": ("mixer", b.mixer),
                             "norm_c": ("norm", a.norm2), "ff_a": ("feed_forward", a.feed_forward),
                             "norm_d": ("norm", b.norm2), "ff_b": ("feed_forward", b.feed_forward)})
    return ModelSpec(width=TW_C, vocab_size=V,
                     embedding=PartSpec("token_embedding", {"vocab_size": V, "width": TW_C}, {"weight": "emb.w"}),
                     position=PartSpec("learned_absolute", {"max_positions": 50, "width": TW_C}, {"weight": "pos.w"}),
                     layers=(layer,), order=(LayerRun(0), LayerRun(0)), final_norm=_norm("nf.", TW_C, EPS),
                     head=PartSpec("linear_head", {"vocab_size": V, "width": TW_C, "tied": True}, {"weight": "emb.w"}),
                     max_positions=50)


def _plain_twice_model(w, ids):
    x = P.plain_embed(torch.tensor(ids), w["emb.w"].double(), w["pos.w"].double())
    for _ in range(2):
        for p in ("L0.", "L1."):
            a, _kv = _pl_attn(_pl_norm(x, w, p + "n1.", EPS), w, p, TW_H, TW_H, 1 / math.sqrt(TW_D), 0)
            x = x + a
        for p in ("L0.", "L1."):
            x = x + _pl_mlp(_pl_norm(x, w, p + "n2.", EPS), w, p)
    return _pl_norm(x, w, "nf.", EPS) @ w["emb.w"].double().t()


@pytest.mark.parametrize("n_req", [1, 3, 40])
def test_two_fused_parts_of_one_kind_in_a_row_keep_their_sums_apart(n_req):
    """Decode steps of few rows through the fused kernels with two attention mixers and two
    feed-forwards one behind the other: the second of a kind adds up the first one's pending sums
    while its workgroups store their own, so the two must not share an array; the logits are the
    plain model's, and the kernel wrapper refuses an output that is the pending sums' array."""
    from mini_gpt_inference_amd.ops import kernels as K, residual as R

    model = DecoderModel(_twice_spec())
    assert model.graph_safe and model.plan_safe
    weights = _random_weights(model, 33)
    _bind(model, weights, "bfloat16")
    rng = np.random.default_rng(n_req)
    steps = 5
    reqs = [rng.integers(0, V, int(rng.integers(1, 7)) + steps).tolist() for _ in range(n_req)]
    want = [_plain_twice_model(weights, ids).numpy() for ids in reqs]
    runner, cache = _runner(model, "bfloat16", num_pages=4 * n_req + 8, max_requests=n_req)
    slots = [cache.acquire_slot() for _ in reqs]
    heads = [len(r) - steps for r in reqs]
    for s, r in zip(slots, reqs):
        assert cache.reserve(s, len(r))
    runner.step(slots, [0] * n_req, heads, sum((r[:h] for r, h in zip(reqs, heads)), []), [])
    seen = []
    launch = K.fused_attention_decode

    def spy(pending, settled, *args, **kwargs):
        out_partials = args[7]
        seen.append((None if pending.partials is None else pending.partials.data_ptr(), out_partials.data_ptr()))
        return launch(pending, settled, *args, **kwargs)

    K.fused_attention_decode = spy
    try:
        for j in range(steps):
            got = runner.step(slots, [h + j for h in heads], [1] * n_req, [r[h + j] for r, h in zip(reqs, heads)],
                              list(range(n_req)))
            ref = np.stack([wv[h + j] for wv, h in zip(want, heads)])
            helpers.assert_close(got, ref, "bfloat16", f"{n_req} requests, decode step {j}")
    finally:
        K.fused_attention_decode = launch
    assert seen, "the fused attention kernel did not run"
    assert all(a != b for a, b in seen)
    if n_req <= 3:      # one token a workgroup: the second mixer reads the first one's sums
        assert any(a is not None for a, _ in seen)
    # and the wrapper itself refuses the shared array
    from mini_gpt_inference_amd.ops.linear import packed_weight

    ff, norm = model.layers[0].parts["ff_a"], model.layers[0].parts["norm_c"]
    n_parts = TW_HID // 64
    x = torch.zeros(n_req, TW_C, device=DEV)
    parts = torch.zeros(n_parts, n_req, TW_C, device=DEV)
    with pytest.raises(K.KernelError, match="pending sums"):
        K.fused_mlp_decode(R.PendingSums(x, parts, n_parts), torch.zeros_like(x), norm.weight, norm.bias, norm.eps,
                           packed_weight(ff.fc_weight), ff.fc_bias, packed_weight(ff.proj_weight), ff.proj_bias,
                           parts, n_req, TW_HID)


# ----------------------------------------------------------------------------- a part that breaks its promise
from mini_gpt_inference_amd.parts.base import register_norm                 # noqa: E402
from mini_gpt_inference_amd.parts.norms import LayerNorm                     # noqa: E402


@register_norm("toy_norm_that_reads_the_host")
class ToyNormThatReadsTheHost(LayerNorm):
    """Promises plan_safe (inherited) and still takes a kernel argument from the host's view of the
    step: its eps grows with the longest sequence.  The results are right whenever its Python runs;
    a plan recorded for the shape would replay the eps of the step it was recorded at."""

    fusable_layer_norm = False

    def forward(self, ctx, x, out, n_rows, rows=None):
        from mini_gpt_inference_amd.ops import kernels as K

        K.layer_norm(x, self.weight, self.bias, out, n_rows, self.eps * ctx.max_seq_len, rows)


def test_plan_verification_names_a_part_that_breaks_its_promise():
    """ModelRunner.verify_plans finds a launcher argument that changed between two steps of one shape."""
    base = _attn_layer(0, C, H, H, D, 0, 1 / math.sqrt(D), HID, EPS)
    lying = PartSpec("toy_norm_that_reads_the_host", {"width": C, "eps": EPS, "bias": True},
                     {"weight": "L0.n2.weight", "bias": "L0.n2.bias"})
    spec = ModelSpec(width=C, vocab_size=V,
                     embedding=PartSpec("token_embedding", {"vocab_size": V, "width": C}, {"weight": "emb.w"}),
                     position=PartSpec("learned_absolute", {"max_positions": 50, "width": C}, {"weight": "pos.w"}),
                     layers=(LayerSpec(base.arrangement, base.norm1, base.mixer, lying, base.feed_forward),),
                     order=(LayerRun(0),), final_norm=_norm("nf.", C, EPS),
                     head=PartSpec("linear_head", {"vocab_size": V, "width": C, "tied": True}, {"weight": "emb.w"}),
                     max_positions=50)
    model = DecoderModel(spec)
    assert model.plan_safe                                   # so it claims
    _bind(model, _random_weights(model, 8), "float32")
    runner, cache = _runner(model, "float32")
    runner.graph_steps = False
    runner.verify_plans = True
    slot = cache.acquire_slot()
    assert cache.reserve(slot, 20)
    runner.step([slot], [0], [4], [1, 2, 3, 4], [3])
    runner.step([slot], [4], [1], [5], [0])                  # shape (1,): recorded
    with pytest.raises(RuntimeError, match="plan_safe.*mgpt_layernorm.*argument"):
        runner.step([slot], [5], [1], [6], [0])              # the same shape one token further: another eps

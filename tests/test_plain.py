"""Pins the plain implementation by what fixes it beside the reference's text: library routines
it must reduce to, invariants, and vectors the reference's own tests hold."""

import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import plain_gpt as P

torch.manual_seed(0)


def test_layer_norm_reduces_to_library():
    x = torch.randn(5, 24, dtype=P.DT) * 3 + 1
    w, b = torch.randn(24, dtype=P.DT), torch.randn(24, dtype=P.DT)
    assert torch.allclose(P.plain_layer_norm(x, w, b, 1e-5), F.layer_norm(x, (24,), w, b, 1e-5), atol=1e-12)
    assert torch.allclose(P.plain_layer_norm(x, w, None, 1e-3), F.layer_norm(x, (24,), w, None, 1e-3), atol=1e-12)


def test_layer_norm_unit_statistics_and_eps_inside_the_root():
    x = torch.randn(3, 64, dtype=P.DT)
    y = P.plain_layer_norm(x, torch.ones(64, dtype=P.DT), None, 0.0)
    assert torch.allclose(y.mean(-1), torch.zeros(3, dtype=P.DT), atol=1e-12)
    assert torch.allclose((y ** 2).mean(-1), torch.ones(3, dtype=P.DT), atol=1e-9)
    # an almost constant row: the result is ruled by eps; eps outside the root would give another value
    row = torch.full((1, 8), 2.0, dtype=P.DT)
    row[0, 0] += 1e-3
    var = ((row - row.mean()) ** 2).mean()
    want = (row - row.mean()) / math.sqrt(var + 1e-2)
    assert torch.allclose(P.plain_layer_norm(row, torch.ones(8, dtype=P.DT), None, 1e-2), want, atol=1e-12)


def test_gelu_is_the_tanh_form():
    u = torch.linspace(-6, 6, 101, dtype=P.DT)
    assert torch.allclose(P.plain_gelu_tanh(u), F.gelu(u, approximate="tanh"), atol=1e-12)
    assert not torch.allclose(P.plain_gelu_tanh(u), F.gelu(u), atol=1e-5)   # the erf form differs
    assert P.plain_gelu_tanh(torch.zeros(1, dtype=P.DT)).item() == 0.0
    assert abs(P.plain_gelu_tanh(torch.tensor([10.0], dtype=P.DT)).item() - 10.0) < 1e-9


def test_linear_and_split_order():
    x = torch.randn(4, 8, dtype=P.DT)
    w, b = torch.randn(24, 8, dtype=P.DT), torch.randn(24, dtype=P.DT)
    assert torch.allclose(P.plain_linear(x, w, b), F.linear(x, w, b), atol=1e-12)
    # rows 0..7 of the fused matrix make q, 8..15 k, 16..23 v; inside each, head i is columns i*D..
    wq, wk, wv = torch.eye(8, dtype=P.DT), 2 * torch.eye(8, dtype=P.DT), 3 * torch.eye(8, dtype=P.DT)
    qkv = P.plain_linear(x, torch.cat([wq, wk, wv]), None)
    q, k, v = P.plain_split_heads(qkv, n_head=2)
    assert q.shape == (2, 4, 4)
    assert torch.equal(q[1], x[:, 4:8]) and torch.equal(k[0], 2 * x[:, 0:4]) and torch.equal(v[1], 3 * x[:, 4:8])


def test_attention_reduces_to_library_sdpa():
    h, t, d = 3, 11, 16
    q, k, v = (torch.randn(h, t, d, dtype=P.DT) for _ in range(3))
    want = F.scaled_dot_product_attention(q[None], k[None], v[None], is_causal=True)[0]
    got = P.plain_causal_attention(q, k, v)
    assert torch.allclose(got, want.transpose(0, 1).reshape(t, h * d), atol=1e-12)
    # without mask: plain softmax(q k^T / sqrt(d)) v
    free = P.plain_causal_attention(q, k, v, causal=False)
    want = torch.softmax(q @ k.transpose(1, 2) / math.sqrt(d), -1) @ v
    assert torch.allclose(free, want.transpose(0, 1).reshape(t, h * d), atol=1e-12)


def test_attention_invariants():
    h, t, d = 2, 9, 8
    q, k, v = (torch.randn(h, t, d, dtype=P.DT) for _ in range(3))
    out = P.plain_causal_attention(q, k, v)
    # the first token sees only itself
    assert torch.allclose(out[0].view(h, d), v[:, 0], atol=1e-12)
    # prefix property: later tokens change nothing before them
    out2 = P.plain_causal_attention(q[:, :5], k[:, :5], v[:, :5])
    assert torch.allclose(out[:5], out2, atol=1e-12)
    # one key/value head shared by all query heads equals repeating it
    shared = P.plain_causal_attention(q, k[:1], v[:1])
    rep = P.plain_causal_attention(q, k[:1].expand(h, t, d), v[:1].expand(h, t, d))
    assert torch.allclose(shared, rep, atol=1e-12)
    # a window only counts distances: the last query over the last w keys alone gives the same
    w = 4
    win = P.plain_causal_attention(q, k, v, window=w)
    tail = P.plain_causal_attention(q[:, -1:], k[:, -w:], v[:, -w:], causal=False)
    assert torch.allclose(win[-1:], tail, atol=1e-12)
    # a wrong scale must show
    assert not torch.allclose(out, P.plain_causal_attention(q, k, v, scale=1.0), atol=1e-3)


def test_embedding_adds_position_rows():
    tok, pos = torch.randn(10, 6, dtype=P.DT), torch.randn(7, 6, dtype=P.DT)
    x = P.plain_embed(torch.tensor([3, 3, 5]), tok, pos)
    assert torch.allclose(x[1] - x[0], pos[1] - pos[0], atol=1e-12)
    assert torch.allclose(x[2], tok[5] + pos[2], atol=1e-12)


def _weights(cfg, seed=0, scale=0.3):
    g = torch.Generator().manual_seed(seed)
    c, f = cfg["n_embd"], 4 * cfg["n_embd"]
    r = lambda *s: torch.randn(*s, generator=g, dtype=P.DT) * scale
    w = {"tok_emb.weight": r(cfg["vocab_size"], c), "pos_emb.weight": r(cfg["block_size"], c),
         "ln_f.weight": 1 + r(c), "ln_f.bias": r(c)}
    for i in range(cfg["n_layer"]):
        p = f"blocks.{i}."
        w.update({p + "ln1.weight": 1 + r(c), p + "ln1.bias": r(c), p + "ln2.weight": 1 + r(c),
                  p + "ln2.bias": r(c), p + "attn.qkv.weight": r(3 * c, c), p + "attn.qkv.bias": r(3 * c),
                  p + "attn.proj.weight": r(c, c), p + "attn.proj.bias": r(c), p + "mlp.fc.weight": r(f, c),
                  p + "mlp.fc.bias": r(f), p + "mlp.proj.weight": r(c, f), p + "mlp.proj.bias": r(c)})
    return w


def test_block_reduces_to_library_pre_norm_layer():
    """A pre-norm library transformer layer with the same tensors must give the same block: a norm
    in the wrong place, a wrong split of the fused projection or the erf GELU would all fail."""
    cfg = {"n_layer": 1, "n_embd": 32, "n_head": 4, "vocab_size": 11, "block_size": 16, "layer_norm_eps": 1e-4}
    w = _weights(cfg)
    layer = torch.nn.TransformerEncoderLayer(32, 4, dim_feedforward=128, dropout=0.0, batch_first=True,
                                             norm_first=True, layer_norm_eps=1e-4,
                                             activation=lambda u: F.gelu(u, approximate="tanh")).double().eval()
    p = "blocks.0."
    with torch.no_grad():
        layer.self_attn.in_proj_weight.copy_(w[p + "attn.qkv.weight"])
        layer.self_attn.in_proj_bias.copy_(w[p + "attn.qkv.bias"])
        layer.self_attn.out_proj.weight.copy_(w[p + "attn.proj.weight"])
        layer.self_attn.out_proj.bias.copy_(w[p + "attn.proj.bias"])
        layer.linear1.weight.copy_(w[p + "mlp.fc.weight"]); layer.linear1.bias.copy_(w[p + "mlp.fc.bias"])
        layer.linear2.weight.copy_(w[p + "mlp.proj.weight"]); layer.linear2.bias.copy_(w[p + "mlp.proj.bias"])
        layer.norm1.weight.copy_(w[p + "ln1.weight"]); layer.norm1.bias.copy_(w[p + "ln1.bias"])
        layer.norm2.weight.copy_(w[p + "ln2.weight"]); layer.norm2.bias.copy_(w[p + "ln2.bias"])
    x = torch.randn(9, 32, dtype=P.DT)
    mask = torch.triu(torch.full((9, 9), float("-inf"), dtype=P.DT), diagonal=1)
    with torch.no_grad():
        want = layer(x[None], src_mask=mask)[0]
    got = P.plain_block(x, w, p, 4, 1e-4)
    assert torch.allclose(got, want, atol=1e-10)


def test_whole_model_is_a_library_encoder_stack_between_embeddings_and_a_tied_head():
    """The whole composition beside the block: torch.nn.TransformerEncoder (pre-norm layers in order,
    then its final norm) fed with the summed embeddings and followed by the tied head is the plain
    forward.  A dropped or misplaced final norm, blocks out of order, a head that is not the token
    table, positions that start at 1: each fails it.  The layers differ from each other (every
    tensor is drawn afresh), so their order shows."""
    cfg = {"n_layer": 3, "n_embd": 48, "n_head": 3, "vocab_size": 29, "block_size": 20, "layer_norm_eps": 1e-3}
    w = _weights(cfg, seed=11)
    def encoder_layer():
        return torch.nn.TransformerEncoderLayer(48, 3, dim_feedforward=192, dropout=0.0, batch_first=True,
                                                norm_first=True, layer_norm_eps=1e-3,
                                                activation=lambda u: F.gelu(u, approximate="tanh"))
    stack = torch.nn.TransformerEncoder(encoder_layer(), num_layers=3, norm=torch.nn.LayerNorm(48, eps=1e-3),
                                        enable_nested_tensor=False).double().eval()
    with torch.no_grad():
        for i, layer in enumerate(stack.layers):
            p = f"blocks.{i}."
            layer.self_attn.in_proj_weight.copy_(w[p + "attn.qkv.weight"])
            layer.self_attn.in_proj_bias.copy_(w[p + "attn.qkv.bias"])
            layer.self_attn.out_proj.weight.copy_(w[p + "attn.proj.weight"])
            layer.self_attn.out_proj.bias.copy_(w[p + "attn.proj.bias"])
            layer.linear1.weight.copy_(w[p + "mlp.fc.weight"]); layer.linear1.bias.copy_(w[p + "mlp.fc.bias"])
            layer.linear2.weight.copy_(w[p + "mlp.proj.weight"]); layer.linear2.bias.copy_(w[p + "mlp.proj.bias"])
            layer.norm1.weight.copy_(w[p + "ln1.weight"]); layer.norm1.bias.copy_(w[p + "ln1.bias"])
            layer.norm2.weight.copy_(w[p + "ln2.weight"]); layer.norm2.bias.copy_(w[p + "ln2.bias"])
        stack.norm.weight.copy_(w["ln_f.weight"]); stack.norm.bias.copy_(w["ln_f.bias"])
    ids = torch.tensor([3, 28, 0, 7, 7, 19, 4, 11, 2])
    x = F.embedding(ids, w["tok_emb.weight"]) + F.embedding(torch.arange(9), w["pos_emb.weight"])
    mask = torch.triu(torch.full((9, 9), float("-inf"), dtype=P.DT), diagonal=1)
    with torch.no_grad():
        want = F.linear(stack(x[None], mask=mask)[0], w["tok_emb.weight"])
    got = P.plain_forward(w, cfg, ids.tolist())
    assert torch.allclose(got, want, atol=1e-9), (got - want).abs().max()
    # the check can fail: the same stack without its final norm, or with two layers swapped, is far off
    stack.norm = None
    with torch.no_grad():
        assert not torch.allclose(F.linear(stack(x[None], mask=mask)[0], w["tok_emb.weight"]), got, atol=1e-3)


def test_forward_head_is_tied_and_prefix_property_holds():
    cfg = {"n_layer": 2, "n_embd": 32, "n_head": 2, "vocab_size": 23, "block_size": 16, "layer_norm_eps": 1e-5}
    w = _weights(cfg, seed=3)
    ids = [1, 5, 22, 0, 7, 7, 3]
    logits = P.plain_forward(w, cfg, ids)
    assert logits.shape == (7, 23)
    assert torch.allclose(P.plain_forward(w, cfg, ids[:4]), logits[:4], atol=1e-12)
    # the head is the embedding matrix: scaling one embedding row scales that logit's matrix row
    x = P.plain_embed(torch.tensor(ids), w["tok_emb.weight"], w["pos_emb.weight"])
    for i in range(2):
        x = P.plain_block(x, w, f"blocks.{i}.", 2, 1e-5)
    x = P.plain_layer_norm(x, w["ln_f.weight"], w["ln_f.bias"], 1e-5)
    assert torch.allclose(logits, F.linear(x, w["tok_emb.weight"]), atol=1e-12)
    with pytest.raises(ValueError, match="block_size"):   # reference tests/test_cache.py:147-158
        P.plain_forward(w, cfg, list(range(17)))


# ------------------------------------------------------------------ sampling (reference tests/test_sampling.py)
def _kept(logits, temperature=1.0, top_k=None, top_p=None):
    """Which ids can be drawn: sweep the uniform number."""
    return sorted({P.plain_sample(np.array(logits, dtype=np.float32), temperature, top_k, top_p, u)[0]
                   for u in np.linspace(0, 0.999999, 4001)})


def test_top_k_vector():
    assert _kept([1.0, 5.0, 3.0, 2.0, 4.0], top_k=2) == [1, 4]           # test_sampling.py:25-30
    rng = np.random.default_rng(0)
    for k in (1, 5, 20):                                                  # test_sampling.py:16-22
        assert P.plain_top_k_mask(rng.normal(size=20), k).sum() == k


def test_top_p_keeps_the_top_token_and_grows_with_p():
    assert _kept([10.0, 0.0, 0.0, 0.0], top_p=1e-6) == [0]               # test_sampling.py:33-38
    lg = np.random.default_rng(1).normal(size=50)
    keep = np.ones(50, dtype=bool)
    small, large = P.plain_top_p_mask(lg, keep, 0.1).sum(), P.plain_top_p_mask(lg, keep, 0.99).sum()
    assert 1 <= small <= large
    # against the reference's own sorted-cumulative rule (sampling.py:55-76) on distinct values
    srt = np.sort(lg)[::-1]
    probs = np.exp(srt - srt.max()); probs /= probs.sum()
    before = np.cumsum(probs) - probs
    assert P.plain_top_p_mask(lg, keep, 0.6).sum() == (before <= 0.6).sum()


def test_temperature_zero_is_argmax_and_the_limit_of_small_temperatures():
    lg = np.random.default_rng(2).normal(size=30).astype(np.float32)
    assert P.plain_sample(lg, 0.0, None, None, 0.7)[0] == int(np.argmax(lg))     # test_sampling.py:49-53
    assert all(P.plain_sample(lg, 1e-4, None, None, u)[0] == int(np.argmax(lg)) for u in (0.0, 0.5, 0.99))
    assert P.plain_sample(np.array([1.0, 3.0, 3.0, 2.0], dtype=np.float32), 0.0, None, None, 0.0)[0] == 1


def test_vocabulary_mask_and_uniform_stream():
    lg = np.zeros(10, dtype=np.float32); lg[8] = 50.0
    assert P.plain_sample(lg, 0.0, None, None, 0.0, real_vocab=8)[0] == 0       # test_reference.py:53-59
    assert all(P.plain_sample(lg, 1.0, None, None, u, real_vocab=8)[0] < 8 for u in np.linspace(0, 0.99, 50))
    us = [P.plain_uniform(7, 3, i) for i in range(2000)]
    assert all(0.0 <= u < 1.0 for u in us) and abs(np.mean(us) - 0.5) < 0.03
    assert P.plain_uniform(7, 3, 5) == P.plain_uniform(7, 3, 5) != P.plain_uniform(7, 4, 5)


def test_inverse_cdf_follows_the_distribution():
    lg = np.array([0.0, math.log(3.0)], dtype=np.float32)    # probabilities 1/4, 3/4
    tok, lo, hi, total = P.plain_sample(lg, 1.0, None, None, 0.2)
    assert tok == 0 and lo == 0.0 and abs(hi / total - 0.25) < 1e-6
    assert P.plain_sample(lg, 1.0, None, None, 0.26)[0] == 1

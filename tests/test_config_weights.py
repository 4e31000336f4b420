"""Configuration, registry, weight loading errors and the random-weights mode (no GPU)."""

import json
import os

import pytest
import torch
from safetensors.torch import load_file, save_file

import helpers
from mini_gpt_inference_amd import GPTConfig
from mini_gpt_inference_amd.config.model_config import ConfigError, read_config_json
from mini_gpt_inference_amd.config.registry import architecture_names, architecture_of, get_architecture
from mini_gpt_inference_amd.weights.loader import WeightError, load_model, strip_prefix
from mini_gpt_inference_amd.weights.random_init import write_random_model


def test_config_round_trip_and_registry(tmp_path):
    cfg = helpers.CONFIGS["B"]
    write_random_model(str(tmp_path), cfg, 1)
    raw = read_config_json(str(tmp_path))
    arch = architecture_of(raw)
    assert arch.name == "gpt2-mini" and "gpt2-mini" in architecture_names()
    assert arch.config_from_json(raw) == cfg
    assert cfg.head_dim == 32
    with pytest.raises(KeyError, match="unknown architecture"):
        get_architecture("no-such-model")


def test_config_errors():
    base = helpers.CONFIGS["A"].to_json_dict()
    with pytest.raises(ConfigError, match="divisible"):
        GPTConfig.from_json_dict({**base, "n_head": 5})
    with pytest.raises(ConfigError, match="lacks required"):
        GPTConfig.from_json_dict({k: v for k, v in base.items() if k != "vocab_size"})
    with pytest.raises(ConfigError, match="does not know"):
        GPTConfig.from_json_dict({**base, "rope_theta": 1e4})
    with pytest.raises(ConfigError, match="positive"):
        GPTConfig.from_json_dict({**base, "n_layer": 0})
    # dropout is read past (reference loader.py:58), model_type names the architecture too
    raw = {k: v for k, v in base.items() if k != "architecture"}
    assert GPTConfig.from_json_dict({**raw, "model_type": "gpt2-mini", "dropout": 0.1}) == helpers.CONFIGS["A"]
    assert GPTConfig.from_json_dict({k: v for k, v in base.items() if k != "layer_norm_eps"}).layer_norm_eps == 1e-5


def test_model_spec_takes_every_size_from_the_config():
    cfg = helpers.CONFIGS["B"]
    spec = get_architecture("gpt2-mini").model_spec(cfg)
    assert len(spec.layers) == 3 and [r.layer for r in spec.order] == [0, 1, 2]
    mixer = spec.layers[0].mixer
    assert mixer.params["n_head"] == 3 and mixer.params["head_dim"] == 32 and mixer.params["bias"] is False
    assert abs(mixer.params["scale"] - 32 ** -0.5) < 1e-12
    assert spec.layers[1].feed_forward.params["hidden"] == 4 * 96
    assert spec.layers[2].norm1.params["eps"] == 1e-6 and "bias" not in spec.layers[2].norm1.weights
    assert spec.head.weights["weight"] == spec.embedding.weights["weight"] == "tok_emb.weight"


def test_random_mode_is_deterministic_and_follows_the_rule(tmp_path):
    cfg = helpers.CONFIGS["A"]
    a = load_file(os.path.join(write_random_model(str(tmp_path / "a"), cfg, 5), "model.safetensors"))
    b = load_file(os.path.join(write_random_model(str(tmp_path / "b"), cfg, 5), "model.safetensors"))
    c = load_file(os.path.join(write_random_model(str(tmp_path / "c"), cfg, 6), "model.safetensors"))
    assert a.keys() == b.keys() and all(torch.equal(a[k], b[k]) for k in a)
    assert not torch.equal(a["tok_emb.weight"], c["tok_emb.weight"])
    assert "lm_head.weight" not in a and a["tok_emb.weight"].dtype == torch.bfloat16
    assert abs(a["tok_emb.weight"].float().std().item() - 0.02) < 0.002
    res = 0.02 / (2 * cfg.n_layer) ** 0.5
    assert abs(a["blocks.0.mlp.proj.weight"].float().std().item() - res) < 0.002
    assert abs(a["blocks.1.ln1.weight"].float().mean().item() - 1.0) < 0.05
    assert a["blocks.0.attn.qkv.bias"].float().abs().max() > 0
    nb = load_file(os.path.join(write_random_model(str(tmp_path / "nb"), helpers.CONFIGS["B"], 1),
                                "model.safetensors"))
    assert not any(k.endswith(".bias") for k in nb)


def test_loader_storage_rule(tmp_path):
    cfg = helpers.CONFIGS["A"]
    d = write_random_model(str(tmp_path / "m"), cfg, 0)
    model, got_cfg, _ = load_model(d, "bfloat16", "cpu")
    attn = model.layers[0].mixer
    assert got_cfg == cfg
    assert attn.qkv_weight.dtype == torch.bfloat16 and attn.qkv_bias.dtype == torch.float32
    assert model.layers[0].norm1.weight.dtype == torch.float32
    assert model.head.weight.data_ptr() == model.embedding.weight.data_ptr()      # one buffer, tied
    model32, _, _ = load_model(d, "float32", "cpu")
    assert model32.layers[0].mixer.qkv_weight.dtype == torch.float32
    # a matrix stored in 32-bit stays 32-bit also when serving in bfloat16
    t = load_file(os.path.join(d, "model.safetensors"))
    t["blocks.0.mlp.fc.weight"] = t["blocks.0.mlp.fc.weight"].float()
    save_file(t, os.path.join(d, "model.safetensors"))
    model, _, _ = load_model(d, "bfloat16", "cpu")
    assert model.layers[0].feed_forward.fc_weight.dtype == torch.float32
    assert model.layers[0].feed_forward.proj_weight.dtype == torch.bfloat16


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    cfg = helpers.CONFIGS["A"]
    d = write_random_model(str(tmp_path / "m"), cfg, 0)
    path = os.path.join(d, "model.safetensors")
    t = load_file(path)
    del t["blocks.1.ln2.bias"]
    del t["ln_f.weight"]
    t["blocks.7.extra"] = torch.zeros(3)
    t["blocks.0.attn.proj.weight"] = torch.zeros(64, 32, dtype=torch.bfloat16)
    save_file(t, path)
    with pytest.raises(WeightError) as exc:
        load_model(d, "float32", "cpu")
    msg = str(exc.value)
    assert "blocks.1.ln2.bias" in msg and "ln_f.weight" in msg and "missing tensors (2)" in msg
    assert "unexpected tensors (1)" in msg and "blocks.7.extra" in msg
    assert "blocks.0.attn.proj.weight should be [64, 64], file has [64, 32]" in msg


def test_bias_tensors_are_required_iff_bias(tmp_path):
    d = write_random_model(str(tmp_path / "m"), helpers.CONFIGS["B"], 1)      # bias = false
    path = os.path.join(d, "model.safetensors")
    t = load_file(path)
    t["blocks.0.attn.qkv.bias"] = torch.zeros(288)
    save_file(t, path)
    with pytest.raises(WeightError, match="unexpected"):
        load_model(d, "float32", "cpu")


def test_prefixes_and_tied_duplicate(tmp_path):
    # reference tests/test_loader.py:18-36
    assert strip_prefix({"module.tok_emb.weight": 1, "module.ln_f.weight": 2}, "module.") == \
        {"tok_emb.weight": 1, "ln_f.weight": 2}
    assert strip_prefix({"tok_emb.weight": 1}, "module.") == {"tok_emb.weight": 1}
    assert strip_prefix({"module.a": 1, "b": 2}, "module.") == {"a": 1, "b": 2}
    cfg = helpers.CONFIGS["A"]
    d = write_random_model(str(tmp_path / "m"), cfg, 0)
    path = os.path.join(d, "model.safetensors")
    t = load_file(path)
    wrapped = {"module._orig_mod." + k: v for k, v in t.items()}
    wrapped["module._orig_mod.lm_head.weight"] = t["tok_emb.weight"].clone()
    save_file(wrapped, path)
    model, _, _ = load_model(d, "float32", "cpu")
    assert model.layers[1].mixer.proj_weight.shape == (64, 64)
    wrapped["module._orig_mod.lm_head.weight"] = t["tok_emb.weight"] * 2
    save_file(wrapped, path)
    with pytest.raises(WeightError, match="one tensor"):
        load_model(d, "float32", "cpu")


def test_missing_files(tmp_path):
    with pytest.raises(ConfigError, match="no config.json"):
        load_model(str(tmp_path), "float32", "cpu")
    with open(tmp_path / "config.json", "w") as fh:
        json.dump(helpers.CONFIGS["A"].to_json_dict(), fh)
    with pytest.raises(WeightError, match="no model.safetensors"):
        load_model(str(tmp_path), "float32", "cpu")


def test_the_models_cost_follows_the_architectures_formulas(tmp_path):
    """DecoderModel.cost() (what bench.py prices a step with) against the GPT-2 formulas written out:
    every matrix, gain and bias once and the tied table once as the head's matrix; the position
    table by row; 12 C^2 matrix elements a token and layer; keys and values of every layer."""
    from mini_gpt_inference_amd.weights.loader import load_model

    cfg = helpers.CONFIGS["A"]
    folder = write_random_model(str(tmp_path / "m"), cfg, 3)
    model, _, _ = load_model(folder, "bfloat16", device="cpu")
    cost = model.cost()
    c, f, L, v, d = cfg.n_embd, 4 * cfg.n_embd, cfg.n_layer, cfg.vocab_size, cfg.head_dim
    matrices = L * (3 * c * c + c * c + 2 * f * c)
    vectors = L * (2 * 2 * c + 3 * c + c + f + c) + 2 * c
    assert cost.run_matrix_elements == matrices and cost.head_matrix_elements == v * c
    assert cost.whole_tensor_bytes == (matrices + v * c) * 2 + vectors * 4
    assert cost.table_row_bytes == c * 2                       # a position's row; the token's row is in the tied matrix
    assert [(r.n_head, r.n_kv_head, r.head_dim, r.window) for r in cost.kv_runs] == [(cfg.n_head, cfg.n_head, d, 0)] * L
    # a decode step of 3 requests that look at 10, 20 and 30 keys
    kv = (10 + 20 + 30) * L * 2 * c * 2
    assert cost.step_read_bytes(3, [10, 20, 30], 2) == cost.whole_tensor_bytes + 3 * c * 2 + kv
    # two whole prompts of 7 and 4 tokens, logits at each one's last token
    attention = sum(4 * (t * (t + 1) // 2) * c for t in (7, 4)) * L
    assert cost.prompt_flops([7, 4], 2) == 2 * 11 * matrices + 2 * 2 * v * c + attention

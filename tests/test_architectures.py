"""Another architecture is an added file: a module dropped into the models package (here a folder
appended to the package's search path, so the tree stays as it is) registers itself, and the
registry, the random-weights mode, the loader, the engine and bench.py work from it with no
other file touched.  The toy architecture below is nobody's model: other config.json keys, other
tensor names, a hidden size of its own, no biases, an untied head."""

import json
import os
import sys
import textwrap

import numpy as np
import pytest
import torch

import plain_gpt as P

TOY_MODULE = textwrap.dedent('''
    """A toy architecture for the tests: pre-norm attention blocks under other names."""
    from dataclasses import asdict, dataclass

    from mini_gpt_inference_amd.config.registry import Architecture, register_architecture
    from mini_gpt_inference_amd.parts.base import PartSpec
    from mini_gpt_inference_amd.parts.model import LayerRun, LayerSpec, ModelSpec


    @dataclass(frozen=True)
    class ToyConfig:
        architecture: str
        depth: int
        dim: int
        heads: int
        ffn: int
        vocab: int
        max_len: int
        eps: float = 1e-5


    def from_json(raw):
        return ToyConfig(**{k: raw[k] for k in ToyConfig.__dataclass_fields__ if k in raw})


    def model_spec(c):
        d = c.dim // c.heads
        norm = lambda name: PartSpec("layer_norm", {"width": c.dim, "eps": c.eps, "bias": False}, {"weight": name})
        layers = []
        for i in range(c.depth):
            p = f"layer{i}/"
            layers.append(LayerSpec(
                PartSpec("pre_norm", {"width": c.dim}), norm(p + "norm_a"),
                PartSpec("paged_causal_attention", {"width": c.dim, "n_head": c.heads, "head_dim": d, "bias": False},
                         {"qkv_weight": p + "qkv", "proj_weight": p + "out"}),
                norm(p + "norm_b"),
                PartSpec("dense_mlp", {"width": c.dim, "hidden": c.ffn, "bias": False},
                         {"fc_weight": p + "up", "proj_weight": p + "down"})))
        return ModelSpec(width=c.dim, vocab_size=c.vocab,
                         embedding=PartSpec("token_embedding", {"vocab_size": c.vocab, "width": c.dim}, {"weight": "tokens"}),
                         position=PartSpec("learned_absolute", {"max_positions": c.max_len, "width": c.dim},
                                           {"weight": "places"}),
                         layers=tuple(layers), order=tuple(LayerRun(i) for i in range(c.depth)),
                         final_norm=norm("norm_out"),
                         head=PartSpec("linear_head", {"vocab_size": c.vocab, "width": c.dim, "tied": False},
                                       {"weight": "unembed"}),
                         max_positions=c.max_len)


    def init_plan(c):
        plan = [("tokens", (c.vocab, c.dim), "normal", 0.1), ("places", (c.max_len, c.dim), "normal", 0.1)]
        for i in range(c.depth):
            p = f"layer{i}/"
            plan += [(p + "norm_a", (c.dim,), "gain", 0.1), (p + "qkv", (3 * c.dim, c.dim), "normal", 0.1),
                     (p + "out", (c.dim, c.dim), "normal", 0.1), (p + "norm_b", (c.dim,), "gain", 0.1),
                     (p + "up", (c.ffn, c.dim), "normal", 0.1), (p + "down", (c.dim, c.ffn), "normal", 0.1)]
        return plan + [("norm_out", (c.dim,), "gain", 0.1), ("unembed", (c.vocab, c.dim), "normal", 0.1)]


    register_architecture(Architecture("toy-renamed", from_json, model_spec, init_plan, asdict))
''')

TOY_JSON = {"architecture": "toy-renamed", "depth": 2, "dim": 96, "heads": 3, "ffn": 160, "vocab": 211,
            "max_len": 80, "eps": 1e-4}


@pytest.fixture(scope="module")
def toy_architecture(tmp_path_factory):
    """The toy module in a folder of its own, which joins the models package's search path."""
    from mini_gpt_inference_amd import models
    from mini_gpt_inference_amd.config import registry

    folder = tmp_path_factory.mktemp("more_models")
    (folder / "toy_renamed.py").write_text(TOY_MODULE)
    models.__path__.append(str(folder))
    try:
        yield registry
    finally:
        models.__path__.remove(str(folder))
        registry._ARCHITECTURES.pop("toy-renamed", None)
        registry._SCANNED.discard("toy_renamed")
        sys.modules.pop("mini_gpt_inference_amd.models.toy_renamed", None)


def _plain_names(tensors, depth):
    """The toy's tensors under the names that the plain implementation reads."""
    names = {"tokens": "tok_emb.weight", "places": "pos_emb.weight", "norm_out": "ln_f.weight"}
    for i in range(depth):
        p, q = f"layer{i}/", f"blocks.{i}."
        names.update({p + "norm_a": q + "ln1.weight", p + "qkv": q + "attn.qkv.weight", p + "out": q + "attn.proj.weight",
                      p + "norm_b": q + "ln2.weight", p + "up": q + "mlp.fc.weight", p + "down": q + "mlp.proj.weight"})
    return {names[k]: v.double() for k, v in tensors.items() if k in names}


def _plain_logits(w, unembed, cfg, ids, rows=None):
    """plain_forward up to the final norm (it multiplies by the token table: here the head is untied)."""
    eps = cfg["layer_norm_eps"]
    x = P.plain_embed(torch.as_tensor(ids), w["tok_emb.weight"], w["pos_emb.weight"])
    for layer in range(cfg["n_layer"]):
        x = P.plain_block(x, w, f"blocks.{layer}.", cfg["n_head"], eps)
    x = P.plain_layer_norm(x, w["ln_f.weight"], None, eps)
    if rows is not None:
        x = x[list(rows)]
    return x @ unembed.t()


def test_a_module_in_the_models_package_is_an_architecture(toy_architecture, tmp_path):
    registry = toy_architecture
    from mini_gpt_inference_amd.config.model_config import read_config_json
    from mini_gpt_inference_amd.parts.model import DecoderModel
    from mini_gpt_inference_amd.weights.loader import WeightError, load_model
    from mini_gpt_inference_amd.weights.random_init import write_random_model

    assert "toy-renamed" in registry.architecture_names() and "gpt2-mini" in registry.architecture_names()
    arch = registry.architecture_of(TOY_JSON)
    cfg = arch.config_from_json(TOY_JSON)
    assert registry.architecture_of_config(cfg) is arch
    folder = write_random_model(str(tmp_path / "toy"), cfg, seed=5)
    assert read_config_json(folder) == TOY_JSON                  # written by the architecture's own conversion
    model, cfg2, arch2 = load_model(folder, "float32", device="cpu")
    assert cfg2 == cfg and arch2 is arch and isinstance(model, DecoderModel)
    cost = model.cost()
    assert cost.run_matrix_elements == 2 * (4 * 96 * 96 + 2 * 96 * 160) and cost.head_matrix_elements == 211 * 96
    assert cost.table_row_bytes == 2 * 96 * 4 and len(cost.kv_runs) == 2       # an untied head: both tables by row
    # the one error of the loader names the toy's own tensors
    from safetensors.torch import load_file, save_file
    tensors = load_file(os.path.join(folder, "model.safetensors"))
    del tensors["layer1/up"]
    save_file(tensors, os.path.join(folder, "model.safetensors"))
    with pytest.raises(WeightError, match="layer1/up"):
        load_model(folder, "float32", device="cpu")
    with pytest.raises(KeyError, match="unknown architecture"):
        registry.get_architecture("no-such-model")
    with pytest.raises(TypeError, match="architecture"):
        registry.architecture_of_config(object())


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_toy_architecture_generates_and_is_benchmarked(toy_architecture, tmp_path, capsys, dtype):
    from safetensors.torch import load_file

    import bench
    import helpers
    from mini_gpt_inference_amd import EngineConfig, SamplingParams
    from mini_gpt_inference_amd.engine.llm_engine import LLMEngine
    from mini_gpt_inference_amd.weights.random_init import write_random_model

    cfg = toy_architecture.architecture_of(TOY_JSON).config_from_json(TOY_JSON)
    folder = write_random_model(str(tmp_path / "toy"), cfg, seed=6)
    tensors = load_file(os.path.join(folder, "model.safetensors"))
    w = _plain_names(tensors, cfg.depth)
    pcfg = {"n_layer": cfg.depth, "n_head": cfg.heads, "layer_norm_eps": cfg.eps}
    engine = LLMEngine.from_folder(folder, EngineConfig(block_size=8, num_blocks=40, max_batch_size=4, dtype=dtype))
    rng = np.random.default_rng(3)
    prompts = [rng.integers(0, cfg.vocab, n).tolist() for n in (3, 17, 30)]
    got = engine.generate(prompts, SamplingParams(max_tokens=12, temperature=0.0))
    assert engine.stats()["graph_steps"] > 0
    for prompt, tokens in zip(prompts, got):
        ids = list(prompt)
        for tok in tokens:
            logits = _plain_logits(w, tensors["unembed"].double(), pcfg, ids, rows=[len(ids) - 1])[0].numpy()
            assert logits[tok] >= logits.max() - 2 * helpers.TOL[dtype] * max(1.0, np.abs(logits).max())
            if dtype == "float32":
                assert tok == int(np.argmax(logits))
            ids.append(tok)
    # bench.py measures it from its config.json alone
    path = tmp_path / "toy.json"
    path.write_text(json.dumps(TOY_JSON))
    capsys.readouterr()
    assert bench.main(["--model-config", str(path), "--steps", "4", "--warmup", "2", "--blocks", "3", "--generate", "20",
                       "--prompt", "9", "--batch", "3", "--kv-block", "8", "--dtype", dtype, "--no-extras"]) == 0
    lines = [line for line in capsys.readouterr().out.splitlines() if line.startswith("{")]
    assert len(lines) == 1
    rec = json.loads(lines[0])
    assert rec["config"]["model"] == "toy-renamed" and rec["config"]["dim"] == 96 and rec["config"]["ffn"] == 160
    assert rec["config"]["head_dim"] == 32 and rec["config"]["mlp_hidden"] == 160 and rec["config"]["seq_len"] == 80
    assert rec["value"] > 0 and rec["blocks"] >= 3 and rec["vs_baseline"] is None
    assert len(rec["config"]) <= 20 and rec["roofline"]["achieved"] > 0

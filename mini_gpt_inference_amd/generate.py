"""Command line in the manner of the reference's scripts: argparse, a config line, the result
(scripts/download_checkpoint.py:19-41 for --max-new-tokens and the sampling defaults
temperature 0.8 / top-k 50; scripts/serve.py:23-33 for --kv-block-size, --num-kv-blocks,
--max-batch-size, --device).  Prompts are token ids: the tokenizer is outside the engine.

    python -m mini_gpt_inference_amd.generate --model DIR --prompt-ids 1,2,3 --max-new-tokens 20
    python -m mini_gpt_inference_amd.generate --random-config cfg.json --seed 0 --prompt-file prompts.txt
"""

from __future__ import annotations

import argparse
import json
import sys
import time
from typing import List

from .config.engine_config import EngineConfig, SamplingParams
from .config.model_config import read_config_json
from .config.registry import architecture_of
from .engine.llm_engine import LLMEngine


def _parse_ids(text: str) -> List[int]:
    return [int(t) for t in text.replace(",", " ").split()]


def build_parser() -> argparse.ArgumentParser:
    ap = argparse.ArgumentParser(prog="mini_gpt_inference_amd.generate", description=__doc__,
                                 formatter_class=argparse.RawDescriptionHelpFormatter)
    src = ap.add_mutually_exclusive_group(required=True)
    src.add_argument("--model", help="folder with config.json and model.safetensors")
    src.add_argument("--random-config", help="a config.json file; weights are drawn from --seed")
    ap.add_argument("--seed", type=int, default=0, help="seed of the random weights and of the sampler")
    prompt = ap.add_mutually_exclusive_group(required=True)
    prompt.add_argument("--prompt-ids", action="append", help="token ids, comma or space separated; repeatable")
    prompt.add_argument("--prompt-file", help="one prompt per line, token ids separated by spaces or commas")
    ap.add_argument("--max-new-tokens", type=int, default=60)
    ap.add_argument("--temperature", type=float, default=0.8, help="0 = greedy")
    ap.add_argument("--top-k", type=int, default=50, help="0 = off")
    ap.add_argument("--top-p", type=float, default=1.0, help="1 = off")
    ap.add_argument("--eot-token-id", type=int, default=None)
    ap.add_argument("--real-vocab-size", type=int, default=None,
                    help="ids at or above it are never sampled (a vocabulary padded for alignment)")
    ap.add_argument("--kv-block-size", type=int, default=16)
    ap.add_argument("--num-kv-blocks", type=int, default=2048)
    ap.add_argument("--max-batch-size", type=int, default=64)
    ap.add_argument("--max-num-batched-tokens", type=int, default=4096)
    ap.add_argument("--prefill-chunk", type=int, default=0, help="0 = whole prompts")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32", "bf16", "fp32"])
    ap.add_argument("--no-graph", action="store_true", help="do not replay decode steps from a HIP graph")
    ap.add_argument("--device", default="cuda")
    return ap


def main(argv=None) -> int:
    args = build_parser().parse_args(argv)
    if args.prompt_ids:
        prompts = [_parse_ids(p) for p in args.prompt_ids]
    else:
        with open(args.prompt_file) as fh:
            prompts = [_parse_ids(line) for line in fh if line.strip()]
    if not prompts or any(not p for p in prompts):
        print("error: every prompt needs at least one token id", file=sys.stderr)
        return 2
    ecfg = EngineConfig(block_size=args.kv_block_size, num_blocks=args.num_kv_blocks,
                        max_batch_size=args.max_batch_size, max_num_batched_tokens=args.max_num_batched_tokens,
                        prefill_chunk=args.prefill_chunk, dtype=args.dtype, use_graph=not args.no_graph,
                        seed=args.seed, real_vocab_size=args.real_vocab_size)
    if args.model:
        engine = LLMEngine.from_folder(args.model, ecfg, args.device)
    else:
        with open(args.random_config) as fh:
            raw = json.load(fh)
        config = architecture_of(raw).config_from_json(raw)
        engine = LLMEngine.from_random(config, args.seed, ecfg, args.device)
    print(f"config: {engine.config}")
    n_params = sum(t.numel() for t in {id(t): t for t in _model_tensors(engine.model)}.values())
    print(f"params: {n_params / 1e6:.1f}M  dtype: {ecfg.dtype}")
    sp = SamplingParams(max_tokens=args.max_new_tokens, temperature=args.temperature,
                        top_k=args.top_k or None, top_p=args.top_p if args.top_p < 1.0 else None)
    start = time.perf_counter()
    outs = engine.generate(prompts, sp, eot_token_id=args.eot_token_id)
    elapsed = time.perf_counter() - start
    for prompt, out in zip(prompts, outs):
        print("prompt:", " ".join(map(str, prompt)))
        print("sample:", " ".join(map(str, out)))
    total = sum(len(o) for o in outs)
    print(f"{total} tokens in {elapsed:.3f} s ({total / max(elapsed, 1e-9):.1f} tok/s), stats: {engine.stats()}")
    return 0


def _model_tensors(model):
    import torch
    for part, _ in model._named_parts():
        for v in vars(part).values():
            if isinstance(v, torch.Tensor):
                yield v


if __name__ == "__main__":
    raise SystemExit(main())

"""Command line in the manner of the reference's ``demo/llama_infer.cpp``.

Reference usage (demo/llama_infer.cpp:128-163):
``llama_infer <checkpoint_path> <tokenizer_path> [device] [--quantize|--no-quantize]`` with
two hard-coded chat turns, 128 new tokens each, temperature 0.8, and a line
``Generated N tokens in Ts (X tokens/s)`` per turn.  Here the first argument is a model
folder (config.json + safetensors); the tokenizer file is optional because prompts may be
given as token ids; what the reference hard-codes is an option.  The device argument is
accepted for compatibility (only ``cuda`` exists); quantisation is not part of this engine.
"""
from __future__ import annotations

import argparse
import sys
import time
from typing import List, Optional

from ..engine import ContinuousBatchEngine, EngineOptions
from ..errors import PhotonError
from ..tokenizer import TikTokenizer
from ..weights import random_model_folder

DEFAULT_TURNS = ["My name is Lummy. Remember that.", "What is my name?"]   # demo/llama_infer.cpp:245,259


def build_parser() -> argparse.ArgumentParser:
    ap = argparse.ArgumentParser(
        prog="llama_infer", description="PhotonInfer-style LLaMA inference demo on one MI355X.")
    ap.add_argument("model_dir", help="model folder (config.json + model.safetensors); with --random-weights: "
                                      "a folder that holds only config.json, or a config.json file")
    ap.add_argument("tokenizer_path", nargs="?", default=None, help="tiktoken-style vocabulary file (optional)")
    ap.add_argument("device", nargs="?", default="cuda", choices=["cuda"], help="only 'cuda' (the GPU) exists")
    ap.add_argument("--random-weights", action="store_true", help="draw weights from --seed instead of reading them")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--weight-std", type=float, default=0.02)
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp32", "bfloat16", "float32"])
    ap.add_argument("--prompt", action="append", default=None, help="prompt text (needs a tokenizer); may repeat")
    ap.add_argument("--prompt-ids", action="append", default=None, help="prompt as comma-separated token ids; may repeat")
    ap.add_argument("--prompt-file", default=None, help="file with one prompt per line (text, or ids with --ids-in-file)")
    ap.add_argument("--ids-in-file", action="store_true")
    ap.add_argument("--max-new-tokens", type=int, default=128)
    ap.add_argument("--temperature", type=float, default=0.8)
    ap.add_argument("--block-size", type=int, default=16)
    ap.add_argument("--num-blocks", type=int, default=None)
    ap.add_argument("--max-batch", type=int, default=32)
    ap.add_argument("--max-step-tokens", type=int, default=2048)
    ap.add_argument("--chunk-size", type=int, default=512)
    ap.add_argument("--max-model-len", type=int, default=None)
    ap.add_argument("--ignore-eos", action="store_true")
    ap.add_argument("--no-quantize", action="store_true", help="accepted and ignored: weights are never quantised")
    return ap


def _model_folder(args) -> str:
    if not args.random_weights:
        return args.model_dir
    out = random_model_folder(args.model_dir, seed=args.seed, std=args.weight_std)
    print(f"Writing random weights (seed {args.seed}) to: {out}")
    return out


def _prompts(args, tok: Optional[TikTokenizer]) -> List[tuple]:
    """(text, ids) pairs."""
    out = []
    for ids in args.prompt_ids or []:
        out.append(("", [int(x) for x in ids.replace(" ", "").split(",") if x]))
    texts = list(args.prompt or [])
    if args.prompt_file:
        with open(args.prompt_file) as f:
            for line in f:
                line = line.strip()
                if not line:
                    continue
                if args.ids_in_file:
                    out.append(("", [int(x) for x in line.replace(",", " ").split()]))
                else:
                    texts.append(line)
    if not out and not texts:
        texts = list(DEFAULT_TURNS)
    if texts and tok is None:
        raise PhotonError("text prompts need a tokenizer file; give <tokenizer_path> or use --prompt-ids")
    for t in texts:
        out.append((t, [tok.bos_id()] + tok.encode(t)))
    return out


def _device_name(args) -> str:
    """What the GPU calls itself (the reference prints its device the same way, demo/llama_infer.cpp)."""
    try:
        import torch
        if torch.cuda.is_available():
            return f"{torch.cuda.get_device_name(0)} (HIP)"
    except Exception:          # the banner must not be what stops the program
        pass
    return "no GPU found"


def main(argv=None) -> int:
    args = build_parser().parse_args(argv)
    print("PhotonInfer - LLaMA Inference Demo")
    print("===================================")
    print(f"Device: {_device_name(args)}")
    print(f"Compute dtype: {args.dtype}\n")
    try:
        tok = None
        if args.tokenizer_path:
            print(f"Loading tokenizer from: {args.tokenizer_path}")
            tok = TikTokenizer.load(args.tokenizer_path)
            print(f"  Vocab size: {tok.vocab_size()}\n")
        model_dir = _model_folder(args)
        print(f"Loading model from: {model_dir}")
        options = EngineOptions(
            dtype=args.dtype, block_size=args.block_size, num_blocks=args.num_blocks, max_batch=args.max_batch,
            max_step_tokens=args.max_step_tokens, chunk_size=args.chunk_size, max_model_len=args.max_model_len,
            seed=args.seed, max_cache_tokens=None if args.num_blocks else 65536)
        engine = ContinuousBatchEngine(model_dir, options)
        cfg = engine.config
        print(f"  Layers: {cfg.num_hidden_layers}")
        print(f"  Dimension: {cfg.hidden_size}\n")
        print("Model ready!\n")
        prompts = _prompts(args, tok)
        start = time.perf_counter()
        ids = [engine.add_request(p, args.max_new_tokens, args.temperature, ignore_eos=args.ignore_eos, prompt=t)
               for t, p in prompts]
        engine.run_until_complete()
        elapsed = time.perf_counter() - start
        total = 0
        for n, (rid, (text, p)) in enumerate(zip(ids, prompts), 1):
            req = engine.get_request(rid)
            gen = req.generated_tokens
            total += len(gen)
            print(f"=== Request {n} ===")
            if text:
                print(f"User: {text}")
            print(f"Prompt tokens: {len(p)}")
            print(f"Generated ids: {','.join(str(t) for t in gen)}")
            if tok is not None:
                shown = [t for t in gen if t != tok.eos_id()]
                print(f"Assistant: {tok.decode(shown)}")
            print(f"Finish reason: {req.finish_reason}\n")
        print(f"Generated {total} tokens in {elapsed:.3f}s ({total / elapsed:.1f} tokens/s)")
        s = engine.get_stats()
        print(f"Steps: {s.num_steps}  Preemptions: {s.num_preemptions}")
    except PhotonError as e:
        print(f"Error: {e}", file=sys.stderr)
        return 1
    return 0


if __name__ == "__main__":
    sys.exit(main())

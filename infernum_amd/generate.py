"""Text (or token-id) generation from the command line, with the options of the
reference's ``generate`` example (infernum-examples/examples/generate.rs:37-86):

    python -m infernum_amd.generate -m MODEL_DIR [PROMPT] [-n 100] [--greedy] [--no-kv-cache]
        [-t 0.7] [-p 0.9] [-s 42] [-r 1.1] [--repetition-penalty-window 64] [--max-seq-len N]

Added here: ``--prompt-ids 1,2,3`` for model folders without a tokenizer (token
ids in, token ids out), ``--random CONFIG.json`` (random weights from a configuration and ``--seed``), ``--dtype bfloat16|float32``, ``--kernels auto|generic``, and the cache's settings
(``--block-size``, ``--num-blocks``, ``--max-batch``, ``--chunk``).  The model class
is chosen by config.json's ``model_type``, as everywhere in the package.
"""
from __future__ import annotations

import argparse
import os
import sys
import time
from typing import List, Optional


def build_parser() -> argparse.ArgumentParser:
    ap = argparse.ArgumentParser(prog="generate", description="Text generation with a model folder "
                                 "(config.json, *.safetensors, optionally tokenizer.json)")
    ap.add_argument("-m", "--model", default=os.environ.get("LLAMA_MODEL_PATH", "models/llama-3.2-1b"),
                    help="path to the model folder (env LLAMA_MODEL_PATH)")
    ap.add_argument("prompt", nargs="?", default="Hello", help="text prompt")
    ap.add_argument("-n", "--max-tokens", type=int, default=100, help="maximum tokens to generate")
    ap.add_argument("--greedy", action="store_true", help="greedy (argmax) decoding instead of sampling")
    ap.add_argument("--no-kv-cache", action="store_true", help="recompute the full sequence each step")
    ap.add_argument("-t", "--temperature", type=float, default=0.7, help="sampling temperature")
    ap.add_argument("-p", "--top-p", type=float, default=0.9, help="nucleus sampling threshold")
    ap.add_argument("-s", "--seed", type=int, default=42, help="RNG seed for sampling")
    ap.add_argument("-r", "--repetition-penalty", type=float, default=1.1,
                    help="repetition penalty factor (1.0 = disabled)")
    ap.add_argument("--repetition-penalty-window", type=int, default=64,
                    help="number of recent tokens considered for the repetition penalty")
    ap.add_argument("--max-seq-len", type=int, default=None,
                    help="longest sequence (prompt and generated tokens); default min(model max, 4096)")
    ap.add_argument("--prompt-ids", default=None, help="comma-separated token ids instead of a text prompt")
    ap.add_argument("--random", metavar="CONFIG.json", default=None,
                    help="no model folder: random weights made from this configuration file and --seed "
                         "(token ids in and out: give --prompt-ids)")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "bf16", "float32", "f32"])
    ap.add_argument("--kernels", default="auto", choices=["auto", "generic"],
                    help="generic: the plain twins of the fast kernels for every product and the attention")
    ap.add_argument("--block-size", type=int, default=16, help="tokens per page of the cache")
    ap.add_argument("--num-blocks", type=int, default=None, help="pages in the pool (default: for max-seq-len)")
    ap.add_argument("--max-batch", type=int, default=32, help="most requests running at once")
    ap.add_argument("--chunk", type=int, default=512, help="longest portion of a prompt in one step")
    return ap


def main(argv: Optional[List[str]] = None) -> int:
    a = build_parser().parse_args(argv)
    from .config import load_config
    from .engine import BatchConfig, Runtime
    from .sampling import GenerateOptions, SamplingParams

    scratch = None
    if a.random is not None:
        # a model folder of random weights (the numbers of ``bin/random_model`` from the same file and seed), made in a
        # temporary folder and loaded like any other; -s is its seed as well as the sampler's
        import tempfile
        import torch
        from . import models  # noqa: F401  (registers the architectures)
        from .config.base import read_config_json
        from .config.registry import config_from_dict
        from .weights import write_random_model
        scratch = tempfile.TemporaryDirectory(prefix="infernum_random_")
        print(f"Random weights from: {a.random} (seed {a.seed})")
        stored = torch.float32 if a.dtype in ("float32", "f32") else torch.bfloat16
        write_random_model(config_from_dict(read_config_json(a.random), where=a.random), scratch.name, a.seed, stored)
        a.model = scratch.name
    print(f"Loading model from: {a.model}")
    config = load_config(a.model)
    max_seq_len = a.max_seq_len or min(getattr(config, "max_position_embeddings", 4096), 4096)
    num_blocks = a.num_blocks or (-(-max_seq_len // a.block_size) + 1)
    bc = BatchConfig(max_batch_size=a.max_batch, max_prefill_tokens=a.chunk, block_size=a.block_size,
                     num_blocks=num_blocks, max_tokens_per_step=max(a.chunk + a.max_batch, 2048))
    rt = Runtime.from_pretrained(a.model, dtype=a.dtype, batch_config=bc, max_seq_len=max_seq_len, kernels=a.kernels)
    print(f"Model loaded ({config.num_hidden_layers} layers, {config.hidden_size} hidden, {config.vocab_size} vocab)")

    sampling = None if a.greedy else SamplingParams(a.temperature, a.top_p, a.seed, a.repetition_penalty,
                                                    a.repetition_penalty_window)
    options = GenerateOptions(max_new_tokens=a.max_tokens, eos_token_id=None, sampling=sampling,
                              use_kv_cache=not a.no_kv_cache)
    if sampling is not None:
        print(f"Sampling: temperature={sampling.temperature}, top_p={sampling.top_p}, seed={sampling.seed}, "
              f"repetition_penalty={sampling.repetition_penalty} (window={sampling.repetition_penalty_window})")
    else:
        print("Decoding: greedy (argmax)")
    print(f"KV cache: {'enabled' if options.use_kv_cache else 'disabled'}")

    if a.prompt_ids is not None:
        prompt = [int(t) for t in a.prompt_ids.replace(" ", "").split(",") if t]
        print("prompt ids:", " ".join(str(t) for t in prompt))
    else:
        if rt.tokenizer is None:
            print(f"error: {a.model} has no tokenizer.json; give --prompt-ids", file=sys.stderr)
            return 2
        prompt = a.prompt
        print(prompt, end="", flush=True)

    t0 = time.perf_counter()
    n = 0
    if options.use_kv_cache:
        for piece in rt.generate_stream(prompt, options):
            n += 1
            print(piece if isinstance(piece, str) else f" {piece}", end="", flush=True)
    else:
        out = rt.generate(prompt, options)
        n = len(out) if not isinstance(out, str) else len(rt.tokenizer.encode(out, add_bos=False))
        print(out if isinstance(out, str) else " " + " ".join(str(t) for t in out), end="")
    dt = time.perf_counter() - t0
    print()
    print(f"Generated {n} tokens in {dt:.2f}s ({n / dt if dt > 0 else 0.0:.1f} tokens/sec)")
    if scratch is not None:
        scratch.cleanup()
    return 0


if __name__ == "__main__":
    sys.exit(main())

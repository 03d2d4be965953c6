"""Generation throughput of a model folder from the command line, in the manner of the reference's
``bench`` example (infernum-examples/examples/bench.rs:70-158): a positional model folder, the number
of tokens to generate (128), ``--dtype bf16|f32``; an 8-token prompt, greedy decoding, one line
"<n> tokens in <s>s = <r> tok/s".  ``--prefill N`` times a prompt of N tokens as well (the reference's
engine bench does that with 512 tokens, bench.rs:1031-1110).  Token ids are seeded random ids.
"""
from __future__ import annotations

import argparse
import random
import sys
import time
from typing import List, Optional


def main(argv: Optional[List[str]] = None) -> int:
    ap = argparse.ArgumentParser(prog="bench", description="generation throughput of a model folder")
    ap.add_argument("model", help="path to the model folder")
    ap.add_argument("n_gen", nargs="?", type=int, default=128, help="number of tokens to generate")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "f32"], help="compute dtype")
    ap.add_argument("--prefill", type=int, default=512, help="also time a prompt of this many tokens (0: skip)")
    ap.add_argument("--kernels", default="auto", choices=["auto", "generic"],
                    help="generic: the plain twins of the fast kernels (slow; for comparisons)")
    ap.add_argument("--gpus", type=int, default=1, help="one GPU only: this engine has no multi-GPU path")
    a = ap.parse_args(argv)
    if a.gpus != 1:
        print("bench: this engine runs on one GPU", file=sys.stderr)
        return 2
    import torch
    from .config import load_config
    from .engine import BatchConfig, Runtime, StepEntry
    from .sampling import GenerateOptions

    config = load_config(a.model)
    dtype = {"bf16": "bfloat16", "f32": "float32"}[a.dtype]
    need = max(a.prefill, 8 + a.n_gen) + 64
    bc = BatchConfig(max_batch_size=4, max_prefill_tokens=max(a.prefill, 512), block_size=16,
                     num_blocks=2 * (need // 16 + 2), max_tokens_per_step=max(a.prefill, 512) + 4)
    rt = Runtime.from_pretrained(a.model, dtype=dtype, batch_config=bc, kernels=a.kernels)
    print(f"Model loaded: {config.num_hidden_layers} layers, {config.hidden_size} hidden, dtype={a.dtype}",
          file=sys.stderr)
    rng = random.Random(0)
    prompt = [rng.randrange(config.vocab_size) for _ in range(8)]
    options = GenerateOptions(max_new_tokens=a.n_gen)
    rt.generate(prompt, GenerateOptions(max_new_tokens=min(8, a.n_gen)))          # warm-up: kernels, graphs
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    out = rt.generate(prompt, options)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    print(f"{len(out)} tokens in {dt:.2f}s = {len(out) / dt:.1f} tok/s")
    if a.prefill > 0:
        ids = [rng.randrange(config.vocab_size) for _ in range(a.prefill)]
        best = None
        for i in range(3):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            rt.engine.step([StepEntry(f"prefill{i}", ids, [a.prefill - 1])])
            torch.cuda.synchronize()
            t = time.perf_counter() - t0
            rt.engine.end(f"prefill{i}")
            if i > 0:
                best = t if best is None else min(best, t)
        print(f"prefill {a.prefill} tokens in {best * 1e3:.2f}ms = {a.prefill / best:.1f} tok/s")
    return 0


if __name__ == "__main__":
    sys.exit(main())

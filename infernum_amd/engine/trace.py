"""Trace replay: given token ids, step by step, through the engine; logits to files.

It samples nothing and has no model code of its own: each step of the trace is
one call of :meth:`Engine.step`, and ``end`` gives a request's pages back through
the engine's cache manager.  The reference has no such tool; the nearest is the
hand-driven loop of infernum-examples/examples/bench.rs:1019-1192.

Input, one JSON object a line:
  {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}
Output: ``OUT/<step>.f32`` (little-endian fp32 [wanted, vocab]) for steps that want
something, and a line ``done <step>`` on standard output after every step.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
from typing import IO, Optional

PAGE_SIZE = 16      # tokens a page; divides the 64 that --max-tokens counts in
MAX_LIVE_REQUESTS = 4


def replay(model_dir: str, dtype: str, out_dir: str, max_tokens: int, stream: IO[str], done: IO[str],
           page_size: int = PAGE_SIZE, poison: bool = False, kernels: str = "auto") -> int:
    from ..cache import CacheConfig
    from .engine import Engine, StepEntry

    os.makedirs(out_dir, exist_ok=True)
    num_pages = max(1, (int(max_tokens) + page_size - 1) // page_size)
    print(f"[trace_run] loading {model_dir} ({dtype}); kernels are compiled on the first call if needed",
          file=sys.stderr, flush=True)
    engine = Engine.from_pretrained(
        model_dir, dtype=dtype,
        cache_config=CacheConfig(page_size=page_size, num_pages=num_pages, num_state_slots=2 * MAX_LIVE_REQUESTS,
                                 poison_freed_pages=poison),
        max_tokens_per_step=max(8192, int(max_tokens)), kernels=kernels)
    print(f"[trace_run] ready: {num_pages} pages of {page_size} tokens", file=sys.stderr, flush=True)
    for line in stream:
        line = line.strip()
        if not line:
            continue
        rec = json.loads(line)
        step = rec["step"]
        entries = [StepEntry(e["id"], e["tokens"], e.get("want", [])) for e in rec.get("entries", [])]
        logits = engine.step(entries)
        if logits.shape[0] > 0:
            arr = logits.detach().to("cpu").numpy().astype("<f4", copy=False)
            tmp = os.path.join(out_dir, f".{step}.f32.tmp")
            arr.tofile(tmp)
            os.replace(tmp, os.path.join(out_dir, f"{step}.f32"))
        for rid in rec.get("end", []):
            engine.end(rid)
        done.write(f"done {step}\n")
        done.flush()
    return 0


def main(argv: Optional[list] = None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description="feed given token ids through a model step by step "
                                 "and write the logits at the wanted places")
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder for <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens live requests hold at any time (each rounded up to a multiple of 64)")
    ap.add_argument("--kernels", default="auto", choices=["auto", "generic"],
                    help="generic: every matrix product and the attention on the plain twins of the fast kernels")
    ap.add_argument("--page-size", type=int, default=PAGE_SIZE, help=argparse.SUPPRESS)
    ap.add_argument("--poison-freed-pages", action="store_true", help=argparse.SUPPRESS)
    a = ap.parse_args(argv)
    return replay(a.model, a.dtype, a.out, a.max_tokens, sys.stdin, sys.stdout, a.page_size, a.poison_freed_pages,
                  a.kernels)


if __name__ == "__main__":
    sys.exit(main())

#!/usr/bin/env python3
"""Decode and prefill throughput of the Llama-3.1-8B shape with random weights on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--layers L]

One "step" is one decode step of the whole batch through the generation loop
(``Runtime.step``): every request brings its last token, the engine runs it
against the paged cache, and the next token is chosen greedily on the device.  Requests start from a 512-token prompt (uniform random
ids), as the reference measures decoding after a prompt
(infernum-examples/examples/bench.rs:1049-1110).  The line printed at the end also
holds the prefill of one 2,048-token prompt, decoding at batch 1 and 64, and the
decode step's place against the HBM roofline.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0                 # MI355X HBM3E, published
PEAK_TFLOPS = {"bf16": 2500.0, "fp32": 157.3}
FP32_CHECK_TOKENS = (96, 64)          # two prompts through the bfloat16 and the 32-bit path of the same model

LLAMA_8B = dict(
    model_type="llama", num_hidden_layers=32, hidden_size=4096, num_attention_heads=32, num_key_value_heads=8,
    intermediate_size=14336, vocab_size=128256, rope_theta=500000.0, rms_norm_eps=1e-5, tie_word_embeddings=False,
    max_position_embeddings=131072,
    rope_scaling=dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                      original_max_position_embeddings=8192),
)
LLAMA_13B = dict(
    model_type="llama", num_hidden_layers=40, hidden_size=5120, num_attention_heads=40, num_key_value_heads=40,
    intermediate_size=13824, vocab_size=32000, rope_theta=10000.0, rms_norm_eps=1e-5, tie_word_embeddings=False,
    max_position_embeddings=4096,
)
CONTEXT_LEN = 4096
PROMPT_LEN = 512
PREFILL_TOKENS = 2048
PAGE_SIZE = 16


def sync():
    import torch
    torch.cuda.synchronize()


def matmul_params(cfg) -> int:
    """Weights that every token multiplies with (embedding gather excluded, head included)."""
    H, I, V = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size
    nh, nkv, d = cfg.num_attention_heads, cfg.num_kv_heads, cfg.head_dim
    per_layer = (nh + 2 * nkv) * d * H + nh * d * H + 3 * H * I
    return cfg.num_hidden_layers * per_layer, V * H


def decode_bytes(cfg, ctx_lens, elem=2) -> float:
    """Bytes a decode step has to read: every weight once, and the keys and values of the live requests."""
    per_layers, head = matmul_params(cfg)
    kv = sum(ctx_lens) * 2 * cfg.num_kv_heads * cfg.head_dim * cfg.num_hidden_layers
    return (per_layers + head + kv) * elem


def prefill_flops(cfg, T) -> float:
    per_layers, head = matmul_params(cfg)
    gemm = 2.0 * T * per_layers + 2.0 * head            # the head runs on one row
    attn = 4.0 * cfg.num_attention_heads * cfg.head_dim * (T * (T + 1) / 2) * cfg.num_hidden_layers
    return gemm + attn


class DecodeRun:
    """B requests through the generation loop itself (scheduler, step function, sampler: ``Runtime``): their
    prompts go in in portions, then every call of ``step`` is one decode step of the whole batch, greedy, the
    tokens chosen on the device (the loop launches a step while the tokens of the one before are still there)."""

    def __init__(self, engine, batch: int, prompt_len: int, new_tokens: int, seed: int = 0):
        import torch
        from infernum_amd import BatchConfig, GenerateOptions, Runtime
        from infernum_amd.engine.scheduler import SequencePhase
        cc = engine.cache.config
        chunk = min(2048, engine.rt.max_tokens_per_step - batch)
        bc = BatchConfig(max_batch_size=batch, max_prefill_tokens=chunk, block_size=cc.page_size,
                         num_blocks=cc.num_pages, max_tokens_per_step=chunk + batch)
        self.engine, self.batch = engine, batch
        self.rt = Runtime(engine, None, bc)
        g = torch.Generator().manual_seed(seed)
        V = engine.spec.vocab_size
        self.seqs = [self.rt.submit(torch.randint(0, V, (prompt_len,), generator=g).tolist(),
                                    GenerateOptions(max_new_tokens=new_tokens)) for _ in range(batch)]
        while any(s.phase != SequencePhase.DECODE for s in self.seqs):
            if any(s.phase == SequencePhase.FINISHED for s in self.seqs):
                raise RuntimeError("a request of the benchmark ended before it decoded: " +
                                   str([s.error or s.finish_reason for s in self.seqs if s.phase == SequencePhase.FINISHED]))
            self.rt.step()
        sync()

    @property
    def ctx(self):
        return [s.num_tokens for s in self.seqs]

    def step(self):
        plan = self.rt.step()
        assert len(plan.decode) == self.batch and not plan.prefill, "a decode step of the whole batch"

    def close(self):
        for s in self.seqs:
            self.rt.scheduler.cancel(s)
        self.rt.run()
        sync()


def prefill_steps(batch: int, prompt_len: int) -> int:
    """Steps the prompts of a batch take to go in (portions of 2,048 tokens): the requests that went in first
    decode meanwhile, so every request is given that many tokens more to generate."""
    return -(-batch * prompt_len // 2048) + 8


def time_decode(engine, batch, steps, warmup, prompt_len=PROMPT_LEN):
    run = DecodeRun(engine, batch, prompt_len, new_tokens=warmup + steps + prefill_steps(batch, prompt_len) + 8)
    for _ in range(warmup):
        run.step()
    sync()
    ctx_mid = [c + steps / 2.0 for c in run.ctx]
    t0 = time.perf_counter()
    for _ in range(steps):
        run.step()
    sync()
    dt = time.perf_counter() - t0
    run.close()
    return dt, ctx_mid


def check_prompts(cfg):
    import torch
    g = torch.Generator().manual_seed(11)
    return [torch.randint(0, cfg.vocab_size, (n,), generator=g).tolist() for n in FP32_CHECK_TOKENS]


def check_logits(engine, cfg):
    """Logits at every place of the check's prompts (one step, two requests), on the host."""
    from infernum_amd.engine import StepEntry
    prompts = check_prompts(cfg)
    logits = engine.step([StepEntry(f"chk{i}", p, list(range(len(p)))) for i, p in enumerate(prompts)])
    for i in range(len(prompts)):
        engine.end(f"chk{i}")
    return logits.float().cpu()


def fp32_check(bf16_logits, cfg, full_layers: int, seed: int) -> dict:
    """The same model (the bfloat16 numbers, widened) through the true 32-bit path: how far the bfloat16 path's
    logits are from it.  (The reference can run the whole model in f32, infernum-examples/examples/bench.rs:97-99.)"""
    import torch
    from infernum_amd import CacheConfig, Engine
    n = sum(FP32_CHECK_TOKENS)
    eng = Engine.from_config(cfg, seed=seed, dtype="float32", stored_as="bfloat16", use_graphs=False,
                             cache_config=CacheConfig(page_size=PAGE_SIZE, num_pages=n // PAGE_SIZE + 4,
                                                      num_state_slots=4))
    ref = check_logits(eng, cfg).double()
    del eng
    torch.cuda.empty_cache()
    diff = (bf16_logits.double() - ref).abs()
    rms = float(ref.pow(2).mean().sqrt())
    return {"layers": cfg.num_hidden_layers, "layers_of_config": full_layers, "tokens": n,
            "max_abs": round(float(diff.max()), 5), "rms_of_logits": round(rms, 5),
            "max_abs_over_rms": round(float(diff.max()) / rms, 5),
            "rms_diff_over_rms": round(float(diff.pow(2).mean().sqrt()) / rms, 5),
            "same_argmax": round(float((bf16_logits.argmax(-1) == ref.argmax(-1)).float().mean()), 4)}


def time_prefill(engine, cfg, dtype: str, repeats: int = 3) -> dict:
    """One prompt of 2,048 tokens in one step, logits at its last place; the best of a few runs after the first."""
    import torch
    from infernum_amd.engine import StepEntry
    g = torch.Generator().manual_seed(7)
    prompt = torch.randint(0, cfg.vocab_size, (PREFILL_TOKENS,), generator=g).tolist()
    best = None
    for i in range(repeats):
        sync()
        t0 = time.perf_counter()
        engine.step([StepEntry(f"p{i}", prompt, [PREFILL_TOKENS - 1])])
        sync()
        t = time.perf_counter() - t0
        engine.end(f"p{i}")
        if i > 0:
            best = t if best is None else min(best, t)
    flops = prefill_flops(cfg, PREFILL_TOKENS)
    return {"value": round(PREFILL_TOKENS / best, 1), "tokens": PREFILL_TOKENS, "ms": round(best * 1e3, 3),
            "frac": round(flops / best / (PEAK_TFLOPS[dtype] * 1e12), 4)}


LLAMA_1B = dict(
    model_type="llama", num_hidden_layers=16, hidden_size=2048, num_attention_heads=32, num_key_value_heads=8,
    head_dim=64, intermediate_size=8192, vocab_size=128256, rope_theta=500000.0, rms_norm_eps=1e-5,
    tie_word_embeddings=True, max_position_embeddings=131072,
    rope_scaling=dict(rope_type="llama3", factor=32.0, low_freq_factor=1.0, high_freq_factor=4.0,
                      original_max_position_embeddings=8192),
)


LLAMA_70B = dict(
    model_type="llama", num_hidden_layers=80, hidden_size=8192, num_attention_heads=64, num_key_value_heads=8,
    intermediate_size=28672, vocab_size=128256, rope_theta=500000.0, rms_norm_eps=1e-5, tie_word_embeddings=False,
    max_position_embeddings=131072,
    rope_scaling=dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                      original_max_position_embeddings=8192),
)


SHAPES = {
    "8b": (LLAMA_8B, "Llama-3-8B", "llama-3.1-8b-shape-random", "llama3(8,1,4,8192) theta 5e5"),
    "13b": (LLAMA_13B, "Llama-2-13B", "llama-2-13b-shape-random", "theta 1e4"),
    "1b": (LLAMA_1B, "Llama-3.2-1B", "llama-3.2-1b-shape-random", "llama3(32,1,4,8192) theta 5e5"),
    # 141 GB of weights in bf16 and 77 GB of second copies of the wide ones: one GPU's memory holds them
    "70b": (LLAMA_70B, "Llama-3.1-70B", "llama-3.1-70b-shape-random", "llama3(8,1,4,8192) theta 5e5"),
}


def serve(a) -> int:
    """Continuous batching of 128 requests on the Llama-3.2-1B shape: prompts of 64 to 2,048 tokens, 32 to 512
    new tokens each (uniform, seeded), greedy, context 4,096.  Prints one JSON line of its own: tokens a second
    (generated, of prompts, together) and the run's place against the roofline (portions of prompts and decoded
    tokens share steps, so they are priced together, step by step; the reference prices prefill and decode apart,
    performance.md:9-41, infernum-examples/examples/bench.rs:1031-1110, where they run apart)."""
    import random
    import torch
    from infernum_amd import BatchConfig, CacheConfig, Engine, GenerateOptions, LlamaConfig, Runtime
    cfg = LlamaConfig.from_dict(LLAMA_1B)
    bc = BatchConfig(max_batch_size=a.serve_batch, max_prefill_tokens=a.serve_chunk, block_size=PAGE_SIZE,
                     num_blocks=a.serve_blocks, max_tokens_per_step=a.serve_budget or max(a.serve_chunk, a.serve_batch))
    engine = Engine.from_config(cfg, seed=0, dtype="bfloat16",
                                cache_config=CacheConfig(page_size=bc.block_size, num_pages=bc.num_blocks,
                                                         num_state_slots=bc.max_batch_size),
                                max_tokens_per_step=bc.max_tokens_per_step)
    rt = Runtime(engine, None, bc, max_seq_len=CONTEXT_LEN)
    rng = random.Random(0)
    jobs = [([rng.randrange(cfg.vocab_size) for _ in range(rng.randint(64, 2048))], rng.randint(32, 512))
            for _ in range(a.serve_requests)]
    # a short warm-up so that kernels are loaded and the common decode shapes are recorded
    rt.generate_batch([j[0][:64] for j in jobs[:4]], GenerateOptions(max_new_tokens=4))
    sync()
    t0 = time.perf_counter()
    seqs = [rt.submit(p, GenerateOptions(max_new_tokens=n)) for p, n in jobs]
    steps = set_back = 0
    # what every step has to do at the least: read every weight once and the keys and values of its requests; two
    # flops per weight and token (the head on the rows that want logits), four per query, key and head dimension
    per_layers, head = matmul_params(cfg)
    kv_bytes_per_token = 2 * cfg.num_kv_heads * cfg.head_dim * cfg.num_hidden_layers * 2
    attn_flops_per_pair = 4.0 * cfg.num_attention_heads * cfg.head_dim * cfg.num_hidden_layers
    total_bytes = total_flops = bound_s = 0.0
    cache = engine.cache
    while not rt.scheduler.is_idle():
        plan = rt.step()
        steps += 1
        set_back += len(plan.set_back)
        if plan.is_empty():
            continue
        keys = pairs = 0.0
        for t in plan.decode:
            keys += t.seq.num_tokens
            pairs += t.seq.num_tokens
        for t in plan.prefill:
            n = len(t.token_ids)
            after = cache.num_tokens(t.seq.id) if cache.has(t.seq.id) else n
            keys += after
            pairs += n * after - n * (n - 1) / 2.0
        rows = len(plan.decode) + sum(1 for t in plan.prefill if t.completes)
        step_bytes = (per_layers + head) * 2.0 + keys * kv_bytes_per_token
        step_flops = 2.0 * per_layers * plan.num_tokens + 2.0 * head * rows + attn_flops_per_pair * pairs
        total_bytes += step_bytes
        total_flops += step_flops
        bound_s += max(step_bytes / (HBM_PEAK_GBS * 1e9), step_flops / (PEAK_TFLOPS["bf16"] * 1e12))
    sync()
    dt = time.perf_counter() - t0
    gen = sum(len(s.generated_ids) for s in seqs)
    prompt = sum(len(j[0]) for j in jobs)
    assert all(s.error is None and len(s.generated_ids) == n for s, (_, n) in zip(seqs, jobs))
    print(json.dumps({"metric": "continuous batching, Llama-3.2-1B shape", "requests": len(jobs),
                      "generated_tokens": gen, "prompt_tokens": prompt, "seconds": round(dt, 3),
                      "generated_tok_per_s": round(gen / dt, 1), "prompt_tok_per_s": round(prompt / dt, 1),
                      "all_tok_per_s": round((gen + prompt) / dt, 1),
                      "roofline": {"bound": "per step the larger of bytes / HBM peak and flops / bf16 peak, summed",
                                   "bound_seconds": round(bound_s, 4), "frac": round(bound_s / dt, 4),
                                   "gb_read_at_least": round(total_bytes / 1e9, 1),
                                   "hbm_frac": round(total_bytes / dt / (HBM_PEAK_GBS * 1e9), 4),
                                   "tflop": round(total_flops / 1e12, 1),
                                   "flops_frac": round(total_flops / dt / (PEAK_TFLOPS["bf16"] * 1e12), 4)},
                      "steps": steps, "ms_per_step": round(dt / steps * 1e3, 3), "set_back": set_back,
                      "graph_replays": engine.graph_replays, "max_batch": bc.max_batch_size,
                      "chunk": bc.max_prefill_tokens, "num_blocks": bc.num_blocks, "dtype": "bf16",
                      "data": "synthetic"}))
    return 0


def long_contexts(a) -> int:
    """Further points of the 8B shape, one JSON line of its own: decode with 16,384 to 131,072 tokens of context
    (Llama-3.1's longest; fewer requests as the contexts grow, so that their prompts go in within seconds), the
    prefill of one prompt of 8,192, 16,384 and 32,768 tokens in a single step, and a prompt of 32,768 tokens going
    in in portions of 8,192 beside eight requests that decode meanwhile."""
    import torch
    from infernum_amd import BatchConfig, CacheConfig, Engine, GenerateOptions, LlamaConfig, Runtime
    from infernum_amd.engine import StepEntry
    from infernum_amd.engine.scheduler import SequencePhase
    cfg = LlamaConfig.from_dict(dict(LLAMA_8B))
    points = ((16384, 8), (32768, 8), (65536, 4), (131072 - 1024, 2))     # the last: up to the model's longest sequence
    tokens = max(b * (c + 64 + prefill_steps(b, c) + 2 * PAGE_SIZE) for c, b in points)
    engine = Engine.from_config(cfg, seed=0, dtype="bfloat16", max_tokens_per_step=32768,
                                cache_config=CacheConfig(page_size=PAGE_SIZE, num_state_slots=10,
                                                         num_pages=tokens // PAGE_SIZE + 8))
    out = {"metric": "long contexts, Llama-3-8B shape", "dtype": "bf16", "data": "synthetic", "decode": {}, "prefill": {},
           "prompt_beside_decoding": {}}
    for ctx_len, batch in points:
        steps = 32
        t_in = time.perf_counter()
        dt, ctx_mid = time_decode(engine, batch, steps, 4, ctx_len)
        gbs = decode_bytes(cfg, ctx_mid) / (dt / steps) / 1e9
        out["decode"][str(ctx_len)] = {"batch": batch, "tokens_per_s": round(batch * steps / dt, 1),
                                       "ms_per_step": round(dt / steps * 1e3, 3), "gb_per_s": round(gbs, 1),
                                       "frac": round(gbs / HBM_PEAK_GBS, 4)}
        print(f"[bench] decode after {ctx_len} tokens x {batch}: {time.perf_counter() - t_in:.1f} s with the prompts",
              file=sys.stderr, flush=True)
    g = torch.Generator().manual_seed(7)
    for T in (8192, 16384, 32768):
        prompt = torch.randint(0, cfg.vocab_size, (T,), generator=g).tolist()
        best = None
        for i in range(3):
            sync()
            t0 = time.perf_counter()
            engine.step([StepEntry(f"long{i}", prompt, [T - 1])])
            sync()
            t = time.perf_counter() - t0
            engine.end(f"long{i}")
            if i > 0:
                best = t if best is None else min(best, t)
        out["prefill"][str(T)] = {"tokens_per_s": round(T / best, 1), "ms": round(best * 1e3, 2),
                                  "frac": round(prefill_flops(cfg, T) / best / (PEAK_TFLOPS["bf16"] * 1e12), 4)}
    # a long prompt in portions beside decoding requests: eight requests decode (512 tokens of context each), then a
    # prompt of 32,768 tokens arrives and goes in 8,192 tokens a step while they go on
    cc = engine.cache.config
    # (the scheduler cuts the portions so that a step holds 8,192 tokens with the decoded ones: the library's products
    # lose a third to half of their rate at 8,200 rows, which fill one tile of 256 more than two rounds of workgroups)
    bc = BatchConfig(max_batch_size=9, max_prefill_tokens=8192, block_size=cc.page_size, num_blocks=cc.num_pages,
                     max_tokens_per_step=8192 + 8)
    rt = Runtime(engine, None, bc)
    V = cfg.vocab_size
    short = [rt.submit(torch.randint(0, V, (PROMPT_LEN,), generator=g).tolist(), GenerateOptions(max_new_tokens=64))
             for _ in range(8)]
    while any(s.phase != SequencePhase.DECODE for s in short):
        rt.step()
    for _ in range(4):
        rt.step()
    big_prompt = torch.randint(0, V, (32768,), generator=g).tolist()
    for attempt in range(2):          # the second time is the one that counts: the first also loads the library's kernels for these rows
        sync()
        before = sum(len(s.generated_ids) + s.pending for s in short)
        t0 = time.perf_counter()
        big = rt.submit(big_prompt, GenerateOptions(max_new_tokens=1))
        steps = 0
        while big.phase != SequencePhase.FINISHED and not big.generated_ids and big.pending == 0:
            rt.step()
            steps += 1
        sync()
        dt = time.perf_counter() - t0
        if attempt == 0:
            rt.scheduler.cancel(big)
            rt.step()
    decoded = sum(len(s.generated_ids) + s.pending for s in short) - before
    flops = prefill_flops(cfg, 32768) + 2.0 * sum(matmul_params(cfg)) * decoded
    out["prompt_beside_decoding"] = {"prompt_tokens": 32768, "tokens_a_step": 8192, "steps": steps, "ms": round(dt * 1e3, 2),
                                     "prompt_tokens_per_s": round(32768 / dt, 1), "decoded_meanwhile": decoded,
                                     "ms_per_step": round(dt / max(steps, 1) * 1e3, 2),
                                     "frac": round(flops / dt / (PEAK_TFLOPS["bf16"] * 1e12), 4)}
    for s in short + [big]:
        rt.scheduler.cancel(s)
    rt.run()
    print(json.dumps(out))
    return 0


def decode_kernels_alone(a) -> int:
    """The kernels that a decode step of the 8B shape spends its time in, alone, on operands of the step's sizes
    at ``--batch`` requests (8 by default; what is in the operands does not change what the kernels do): the
    product with each of a layer's four weights by the kernel that the routes of ``parts/linear.py`` give these
    rows (at 8 rows the weight-streaming kernel, the gate+up matrix in the layout made for it; at 64 the LDS-tiled
    kernel with K split over workgroups, or with the activation in its epilogue), and the attention over 527
    cached tokens with the rotation and the write of the token's key and value inside.  For hardware counters
    (``rocprofv3 --pmc ... -- python3 bench.py --decode-kernels``): nothing else runs on the GPU, no library kernel
    either (the operands are uninitialised memory; tables and positions come from the host by copies)."""
    import math
    import torch
    from infernum_amd.kernels import api as K
    cfg = dict(LLAMA_8B)
    H, I, nh, nkv = cfg["hidden_size"], cfg["intermediate_size"], cfg["num_attention_heads"], cfg["num_key_value_heads"]
    d, B, ctx, dev = H // nh, a.batch, PROMPT_LEN + 15, "cuda:0"
    bf = dict(dtype=torch.bfloat16, device=dev)
    weights = [("qkv", (nh + 2 * nkv) * d, H, None), ("o", H, nh * d, None), ("gate_up", 2 * I, H, "swiglu"), ("down", H, I, None)]
    x = {Kd: torch.empty((B, Kd), **bf) for _, _, Kd, _ in weights}
    pages_per = -(-(ctx + 1) // PAGE_SIZE)
    kp = torch.empty((B * pages_per, nkv, PAGE_SIZE, d), **bf)
    vp = torch.empty((B * pages_per, nkv, d, PAGE_SIZE), **bf)
    bt = torch.arange(B * pages_per, dtype=torch.int32).reshape(B, pages_per).to(dev)
    pos = torch.full((B,), ctx, dtype=torch.int32).to(dev)
    slots = (torch.arange(B, dtype=torch.int32) * pages_per * PAGE_SIZE + ctx).to(dev)
    inv_freq = (500000.0 ** (-torch.arange(0, d, 2, dtype=torch.float64) / d)).to(dev)
    out = torch.empty((B, nh * d), **bf)
    times = {}
    import importlib
    L = importlib.import_module("infernum_amd.parts.linear")
    from infernum_amd.parts.base import Runtime
    rt = Runtime(torch.device(dev), torch.bfloat16)
    for name, N, Kd, epilogue in weights:
        w = torch.empty((N, Kd), **bf)
        L.prepare_weights(rt, [(w, epilogue, epilogue is None)])        # the copy in the weight-streaming kernel's layout
        for _ in range(a.warmup):
            L.linear(x[Kd], w, epilogue=epilogue, keep_split=epilogue is None)
        sync()
        t0 = time.perf_counter()
        for _ in range(a.steps):
            y = L.linear(x[Kd], w, epilogue=epilogue, keep_split=epilogue is None)
        sync()
        times[name] = round((time.perf_counter() - t0) / a.steps * 1e6, 1)
        if name == "qkv":
            qkv = y                      # the partial sums of the QKV product: what the attention kernel reads
    for i in range(a.warmup + a.steps):
        if i == a.warmup:
            sync()
            t0 = time.perf_counter()
        K.attention_decode_rotating(qkv, pos, inv_freq, d, slots, kp, vp, out, bt, nh, nkv, d, 1.0 / math.sqrt(d), 0, ctx + 1)
    sync()
    times["attention"] = round((time.perf_counter() - t0) / a.steps * 1e6, 1)
    print(json.dumps({"metric": "decode kernels alone, Llama-3-8B shape", "batch": B, "context": ctx,
                      "us_per_call_from_the_host": times}))
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=240)      # 16 + 240 = the 256 generated tokens of the workload
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the configuration has (both are reported)")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    ap.add_argument("--no-points", action="store_true", help="skip batch 1 / 64 and the prefill")
    ap.add_argument("--prefill-only", action="store_true",
                    help="only the prefill of 2,048 tokens, a few times (for profiles); prints its record alone")
    ap.add_argument("--shape", default="8b", choices=sorted(SHAPES),
                    help="8b: Llama-3.1-8B (the default, the headline); 13b: Llama-2-13B (40 key/value heads); "
                         "1b: Llama-3.2-1B (heads of 64, tied head); 70b: Llama-3.1-70B (all 80 layers on the one GPU; give "
                         "--no-fp32-check, the 32-bit twin does not fit beside it)")
    ap.add_argument("--points", default="1,64", help="batches of the further decode points, e.g. 1,64,128,256")
    ap.add_argument("--prompt-len", type=int, default=PROMPT_LEN, help="tokens of every request's prompt")
    ap.add_argument("--peaks", action="store_true",
                    help="only measure this GPU's streaming read bandwidth and bf16 matrix rate; a JSON line of its own")
    ap.add_argument("--long", action="store_true",
                    help="decode at 16k and 32k tokens of context and prefills of 8k and 16k tokens instead (a JSON line of its own)")
    ap.add_argument("--no-fp32-check", action="store_true", help="skip the comparison with the 32-bit path")
    ap.add_argument("--decode-kernels", action="store_true",
                    help="only the decode step's two kernels on operands of the 8B shape (for hardware counters)")
    ap.add_argument("--serve", action="store_true",
                    help="continuous batching of 128 requests on the 1B shape instead (a JSON line of its own)")
    ap.add_argument("--serve-requests", type=int, default=128)
    ap.add_argument("--serve-batch", type=int, default=128)
    ap.add_argument("--serve-chunk", type=int, default=2048)
    ap.add_argument("--serve-budget", type=int, default=0,
                    help="tokens of a step, decoded ones and portions together (default: the larger of chunk and batch: a step of\n"
                         "2,048 rows fills the library's tiles of 256, one of 2,100 pays for 2,304)")
    ap.add_argument("--serve-blocks", type=int, default=16384)
    a = ap.parse_args()
    if a.gpus != 1:
        print(f"bench.py measures one GPU: this engine has no multi-GPU path (asked for --gpus {a.gpus})")
        return 2

    if a.decode_kernels:
        return decode_kernels_alone(a)
    if a.serve:
        return serve(a)
    if a.long:
        return long_contexts(a)
    if a.peaks:
        from infernum_amd.peaks import measure
        print(json.dumps(measure()))
        return 0
    import torch
    from infernum_amd import CacheConfig, Engine, LlamaConfig

    raw = dict(SHAPES[a.shape][0])
    point_batches = [int(b) for b in a.points.split(",") if b] if not a.no_points else []
    full_layers = raw["num_hidden_layers"]
    if a.layers:
        raw["num_hidden_layers"] = a.layers
    cfg = LlamaConfig.from_dict(raw)
    dtype = {"bf16": "bfloat16", "fp32": "float32"}[a.dtype]
    elem = 2 if a.dtype == "bf16" else 4
    max_batch = 1 if a.prefill_only else max([a.batch] + point_batches)
    tokens_needed = max(max_batch * (a.prompt_len + a.steps + a.warmup + prefill_steps(max_batch, a.prompt_len)
                                     + 2 * PAGE_SIZE), PREFILL_TOKENS + PAGE_SIZE)
    t_load = time.perf_counter()
    engine = Engine.from_config(cfg, seed=0, dtype=dtype,
                                cache_config=CacheConfig(page_size=PAGE_SIZE,
                                                         num_pages=tokens_needed // PAGE_SIZE + max_batch,
                                                         num_state_slots=max_batch + 1),
                                max_tokens_per_step=8192)
    sync()
    print(f"[bench] model ready in {time.perf_counter() - t_load:.1f} s", file=sys.stderr, flush=True)

    if a.prefill_only:
        print(json.dumps({"prefill": time_prefill(engine, cfg, a.dtype, repeats=max(3, a.warmup))}))
        return 0

    import importlib
    gemm_route = importlib.import_module("infernum_amd.parts.linear").gemm_routes()["route"]
    # ---- the timed K steps at the headline batch ---------------------------------
    dt, ctx_mid = time_decode(engine, a.batch, a.steps, a.warmup, a.prompt_len)
    ms_per_step = dt / a.steps * 1e3
    value = a.batch * a.steps / dt
    achieved = decode_bytes(cfg, ctx_mid, elem) / (dt / a.steps) / 1e9
    out = {
        "metric": f"decode tok/s @ batch {a.batch}, {SHAPES[a.shape][1]} shape", "value": round(value, 2), "unit": "tokens/s",
        "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": a.dtype, "data": "synthetic",
        "config": {
            "model": SHAPES[a.shape][2], "layers": cfg.num_hidden_layers, "layers_of_config": full_layers,
            "hidden_size": cfg.hidden_size, "num_heads": cfg.num_attention_heads, "num_kv_heads": cfg.num_kv_heads,
            "head_dim": cfg.head_dim, "intermediate_size": cfg.intermediate_size, "vocab_size": cfg.vocab_size,
            "global_batch": a.batch, "prompt_len": a.prompt_len, "seq_len": CONTEXT_LEN, "page_size": PAGE_SIZE,
            "parallelism": "none", "sampling": "greedy", "gemm_route": gemm_route,
            "rope": SHAPES[a.shape][3],
        },
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4)},
    }

    if not a.no_points:
        points = {}
        for b in point_batches:
            steps = max(16, min(a.steps, 64))
            d, ctx_b = time_decode(engine, b, steps, max(4, min(a.warmup, 8)), a.prompt_len)
            points[f"decode_b{b}"] = round(b * steps / d, 2)
            if b > 64:          # the further points carry their place against the roofline with them
                points[f"decode_b{b}_hbm_frac"] = round(decode_bytes(cfg, ctx_b, elem) / (d / steps) / 1e9 / HBM_PEAK_GBS, 4)
        out["points"] = points
        out["prefill"] = time_prefill(engine, cfg, a.dtype)
        # the same fractions against what a bare stream of loads and a bare chain of matrix instructions reach here
        from infernum_amd.peaks import measure
        peaks = measure()
        out["roofline"]["measured_peak"] = peaks["hbm_read_gbs"]
        out["roofline"]["frac_of_measured"] = round(achieved / peaks["hbm_read_gbs"], 4)
        if a.dtype == "bf16":
            out["prefill"]["measured_peak_tflops"] = peaks["bf16_mfma_tflops"]
            out["prefill"]["frac_of_measured"] = round(
                out["prefill"]["frac"] * PEAK_TFLOPS["bf16"] / peaks["bf16_mfma_tflops"], 4)
        if a.dtype == "bf16" and not a.no_fp32_check:
            logits = check_logits(engine, cfg)
            del engine
            torch.cuda.empty_cache()
            out["fp32_check"] = fp32_check(logits, cfg, full_layers, seed=0)
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())

"""Generation through the entry points on the GPU: greedy tokens against the plain
implementation, sampled tokens against the plain sampler fed with the engine's logits,
continuous batching with portions and with too few pages, the command line."""
import os
import subprocess
import sys

import pytest
import torch

import plain_llama as P
import tiny_models as TM

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    out = {}
    for name in ("A", "B"):
        d = str(tmp_path_factory.mktemp(f"gen{name}"))
        TM.write_tiny(name, d, dtype=torch.float32)
        out[name] = (d,) + P.read_model(d)
    return out


def _runtime(d, dtype, **kw):
    from infernum_amd import BatchConfig, Runtime
    return Runtime.from_pretrained(d, dtype=dtype, batch_config=BatchConfig(**kw))


def test_greedy_A_through_the_entry_point(folders):
    """Configuration A's workload: one prompt of 7 tokens, 16 greedy tokens, pages of 4."""
    from infernum_amd import GenerateOptions
    d, cfg, w = folders["A"]
    prompt = [3, 141, 59, 26, 53, 58, 97]
    want = P.greedy(cfg, w, prompt, 16, eos=cfg["eos_token_id"])     # the entry point stops at the model's own
    assert len(want) == 16
    rt = _runtime(d, "float32", block_size=4, num_blocks=16, max_batch_size=2)
    assert rt.generate(prompt, GenerateOptions(max_new_tokens=16)) == want
    assert list(rt.generate_stream(prompt, GenerateOptions(max_new_tokens=16))) == want
    assert rt.generate(prompt, GenerateOptions(max_new_tokens=5, use_kv_cache=False)) == want[:5]
    # the end-of-sequence token stops and is not emitted
    assert rt.generate(prompt, GenerateOptions(max_new_tokens=16, eos_token_id=want[6])) == want[:want.index(want[6])]
    assert rt.engine.cache.free_pages() == 16


@pytest.mark.parametrize("dtype", ["float32"])
def test_greedy_B_varied_tokens(folders, dtype):
    """A's tied head mostly repeats the last token; B's separate head gives a varied continuation,
    which a fault in the cache or the positions would change."""
    from infernum_amd import GenerateOptions
    d, cfg, w = folders["B"]
    prompt = [3, 141, 59, 26, 53, 58, 97]
    want = P.greedy(cfg, w, prompt, 24, eos=cfg["eos_token_id"])
    assert len(set(want)) >= 5
    rt = _runtime(d, dtype, block_size=8, num_blocks=8, max_batch_size=2, max_prefill_tokens=4)
    assert rt.generate(prompt, GenerateOptions(max_new_tokens=24)) == want


def test_sampled_B_portions_mixed_with_decoding(folders):
    """Configuration B's workload: prompts of 5, 13 and 29 tokens, portions of 8 beside decoded tokens,
    temperature 0.7 with a fixed seed, 12 new tokens each, pages of 8.  The engine's tokens must be the
    plain sampler's tokens on the plain model's logits of the same history."""
    from infernum_amd import GenerateOptions, SamplingParams
    d, cfg, w = folders["B"]
    g = torch.Generator().manual_seed(3)
    prompts = [torch.randint(0, cfg["vocab_size"], (n,), generator=g).tolist() for n in (5, 13, 29)]
    sp = [SamplingParams(temperature=0.7, top_p=0.9, seed=100 + i, repetition_penalty=1.1,
                         repetition_penalty_window=8) for i in range(3)]
    rt = _runtime(d, "float32", block_size=8, num_blocks=24, max_batch_size=3, max_prefill_tokens=8,
                  max_tokens_per_step=16)
    sizes, real_step = [], rt.engine.step
    rt.engine.step = lambda entries, **kw: (sizes.append(sorted(len(e.tokens) for e in entries)),
                                            real_step(entries, **kw))[1]
    got = rt.generate_batch(prompts, [GenerateOptions(max_new_tokens=12, sampling=s) for s in sp])
    assert any(e[0] == 1 and e[-1] > 1 for e in sizes), f"no step mixed decoded tokens with a portion: {sizes}"
    assert max(sum(e) for e in sizes) <= 16 and max(max(e) for e in sizes) <= 8
    for p, s, out in zip(prompts, sp, got):
        toks = list(p)
        for i in range(12):
            logits = P.forward(cfg, w, toks)[-1]
            u = P.uniform_for_token(s.seed, i)
            want = P.sample_token(logits, s.temperature, s.top_p, u, s.repetition_penalty, toks[-8:])
            if want == cfg["eos_token_id"]:                 # the model's end-of-sequence token stops the request
                assert len(out) == i
                break
            assert i < len(out) and want == out[i], f"request with seed {s.seed}: token {i}: the plain sampler gives {want}"
            toks.append(want)
        else:
            assert len(out) == 12


def test_too_few_pages_changes_no_greedy_token(folders):
    from infernum_amd import GenerateOptions
    d, cfg, w = folders["A"]
    g = torch.Generator().manual_seed(5)
    prompts = [torch.randint(0, 256, (n,), generator=g).tolist() for n in (9, 17, 6, 12)]
    eos = cfg["eos_token_id"]
    want = [P.greedy(cfg, w, p, 20, eos=eos) for p in prompts]
    roomy = _runtime(d, "float32", block_size=4, num_blocks=64, max_batch_size=4, max_prefill_tokens=8)
    assert roomy.generate_batch(prompts, GenerateOptions(max_new_tokens=20)) == want
    tight = _runtime(d, "float32", block_size=4, num_blocks=18, max_batch_size=4, max_prefill_tokens=8)
    seqs = [tight.submit(p, GenerateOptions(max_new_tokens=20, eos_token_id=eos)) for p in prompts]
    n_back = 0
    while not tight.scheduler.is_idle():
        n_back += len(tight.step().set_back)
    assert [s.generated_ids for s in seqs] == want
    assert n_back > 0, "the pool was meant to run out"
    tight.scheduler.reap(tight.engine.cache)
    tight.engine.cache.check()
    assert tight.engine.cache.free_pages() == 18


def _record_logits(rt):
    """Wraps the engine's step function: (request, place) -> the logits row that came back for it."""
    seen, real_step = {}, rt.engine.step

    def step(entries, **kw):
        before = {e.request: (rt.engine.cache.num_tokens(e.request) if rt.engine.cache.has(e.request) else 0)
                  for e in entries}
        logits = real_step(entries, **kw)
        rows = logits.detach().double().cpu()
        k = 0
        for e in entries:
            for wanted in e.want:
                seen.setdefault(e.request, {})[before[e.request] + wanted] = rows[k]
                k += 1
        assert k == rows.shape[0]
        return logits
    rt.engine.step = step
    return seen


@pytest.mark.parametrize("num_blocks", [64, 14])
def test_bfloat16_generation_through_the_scheduler_token_by_token(tmp_path, num_blocks):
    """Greedy generation in bfloat16 through scheduler, step function and sampler, prompts in portions beside
    decoded tokens (and, with 14 pages, requests set back and computed again): at every place where a token was
    chosen the engine's logits are the plain model's for the same history within the bfloat16 tolerance, the
    token is the first largest of the engine's logits, and its plain logit is within twice the tolerance of the
    plain model's largest."""
    from infernum_amd import GenerateOptions
    TOL = 6e-2
    d = TM.write_tiny("B", str(tmp_path / "B16"), dtype=torch.bfloat16)
    cfg, w = P.read_model(d)
    g = torch.Generator().manual_seed(8)
    prompts = [torch.randint(0, cfg["vocab_size"], (n,), generator=g).tolist() for n in (21, 9, 33, 14)]
    rt = _runtime(d, "bfloat16", block_size=8, num_blocks=num_blocks, max_batch_size=4, max_prefill_tokens=8,
                  max_tokens_per_step=16)
    seen = _record_logits(rt)
    seqs = [rt.submit(p, GenerateOptions(max_new_tokens=18)) for p in prompts]
    n_back = 0
    while not rt.scheduler.is_idle():
        n_back += len(rt.step().set_back)
    assert (n_back > 0) == (num_blocks == 14), f"{n_back} requests were set back with {num_blocks} pages"
    worst = 0.0
    for s, p in zip(seqs, prompts):
        out = list(s.generated_ids)
        assert len(out) == 18 and s.error is None
        ref = P.forward(cfg, w, p + out)
        for i, t in enumerate(out):
            place = len(p) + i - 1
            row = seen[s.id][place]                       # after a set-back: the row computed last for the place
            rms = ref[place].pow(2).mean().sqrt()
            worst = max(worst, float((row - ref[place]).abs().max() / rms))
            assert int(torch.argmax(row)) == t
            assert float((ref[place].max() - ref[place][t]) / rms) <= 2 * TOL
    print(f"bfloat16 generation with {num_blocks} pages: worst |diff| / rms {worst:.2e}, {n_back} set back")
    assert worst <= TOL
    rt.scheduler.reap(rt.engine.cache)
    rt.engine.cache.check()
    assert rt.engine.cache.free_pages() == num_blocks


def test_too_few_pages_changes_no_sampled_token(folders):
    """Sampled requests that are set back and computed again draw the same tokens: the draw is keyed by the
    seed and the number of tokens generated so far, and the logits of a history do not depend on how it was
    computed.  Against the plain sampler on the plain model's logits as well."""
    from infernum_amd import GenerateOptions, SamplingParams
    d, cfg, w = folders["B"]
    g = torch.Generator().manual_seed(6)
    prompts = [torch.randint(0, cfg["vocab_size"], (n,), generator=g).tolist() for n in (9, 17, 6, 12)]
    sp = [SamplingParams(temperature=0.8, top_p=0.95, seed=7 + i, repetition_penalty=1.05,
                         repetition_penalty_window=6) for i in range(4)]
    opts = [GenerateOptions(max_new_tokens=16, sampling=s, eos_token_id=cfg["vocab_size"] - 1) for s in sp]
    roomy = _runtime(d, "float32", block_size=4, num_blocks=64, max_batch_size=4, max_prefill_tokens=8)
    want = roomy.generate_batch(prompts, opts)
    assert all(len(out) == 16 for out in want), "a request stopped at its end-of-sequence token: take another"
    tight = _runtime(d, "float32", block_size=4, num_blocks=17, max_batch_size=4, max_prefill_tokens=8)
    seqs = [tight.submit(p, o) for p, o in zip(prompts, opts)]
    n_back = 0
    while not tight.scheduler.is_idle():
        n_back += len(tight.step().set_back)
    assert n_back > 0, "the pool was meant to run out"
    assert [list(s.generated_ids) for s in seqs] == want
    for p, s, out in zip(prompts, sp, want):
        toks = list(p)
        for i, t in enumerate(out):
            u = P.uniform_for_token(s.seed, i)
            assert P.sample_token(P.forward(cfg, w, toks)[-1], s.temperature, s.top_p, u, s.repetition_penalty,
                                  toks[-6:]) == t
            toks.append(t)
    tight.scheduler.reap(tight.engine.cache)
    tight.engine.cache.check()
    assert tight.engine.cache.free_pages() == 17


def test_command_line(folders):
    d, cfg, w = folders["A"]
    prompt = [3, 141, 59, 26, 53, 58, 97]
    want = P.greedy(cfg, w, prompt, 6, eos=cfg["eos_token_id"])
    assert len(want) == 6
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "generate"), "-m", d, "--greedy", "-n", "6",
                           "--dtype", "float32", "--prompt-ids", ",".join(map(str, prompt)), "--max-seq-len", "64"],
                          capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-3000:]
    assert "Decoding: greedy (argmax)" in proc.stdout and "KV cache: enabled" in proc.stdout
    assert " ".join(map(str, want)) in proc.stdout
    assert "Generated 6 tokens in" in proc.stdout


def test_command_line_with_random_weights(folders, tmp_path):
    """--random CONFIG.json --seed S: the tokens of the folder that bin/random_model writes from the same two."""
    import json
    d, cfg, w = folders["B"]
    config = tmp_path / "config.json"
    config.write_text(json.dumps(cfg))
    from infernum_amd.config import LlamaConfig
    from infernum_amd.weights import write_random_model
    folder = write_random_model(LlamaConfig.from_dict(cfg, where="B"), str(tmp_path / "model"), 9, torch.float32)
    pcfg, pw = P.read_model(folder)
    prompt = [3, 141, 59, 26, 53]
    want = P.greedy(pcfg, pw, prompt, 6, eos=pcfg["eos_token_id"])
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "generate"), "--random", str(config), "-s", "9",
                           "--greedy", "-n", "6", "--dtype", "float32", "--prompt-ids", ",".join(map(str, prompt)),
                           "--max-seq-len", "64"], capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-3000:]
    assert "Random weights from:" in proc.stdout and " ".join(map(str, want)) in proc.stdout


def test_bench_command_line(folders):
    d, cfg, w = folders["B"]
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "bench"), d, "12", "--dtype", "f32",
                           "--prefill", "40"], capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-3000:]
    assert "12 tokens in" in proc.stdout and "tok/s" in proc.stdout and "prefill 40 tokens" in proc.stdout
    assert "Model loaded: 3 layers, 128 hidden, dtype=f32" in proc.stderr


@pytest.mark.parametrize("num_blocks", [64, 13])
def test_one_step_ahead_changes_no_token(folders, num_blocks):
    """With look-ahead a step is launched while the tokens of the step before it are still on the device; the
    requests get the same tokens as when every step waits for its tokens: greedy and sampled requests, one that
    stops at an end-of-sequence token (its row in the step launched meanwhile is wasted, not wrong), one of a
    single new token, prompts in portions, and (13 pages) requests set back with a token still on the way."""
    from infernum_amd import GenerateOptions, SamplingParams
    d, cfg, w = folders["B"]
    g = torch.Generator().manual_seed(12)
    prompts = [torch.randint(0, cfg["vocab_size"], (n,), generator=g).tolist() for n in (9, 17, 6, 12, 5)]
    probe = _runtime(d, "float32", block_size=4, num_blocks=64, max_batch_size=6, max_prefill_tokens=8)
    probe.look_ahead = False
    free_run = probe.generate(prompts[1], GenerateOptions(max_new_tokens=16))
    eos = free_run[9]                                          # request 1 stops where this token first comes
    opts = [GenerateOptions(max_new_tokens=16),
            GenerateOptions(max_new_tokens=16, eos_token_id=eos),
            GenerateOptions(max_new_tokens=14, sampling=SamplingParams(temperature=0.8, top_p=0.9, seed=3,
                                                                       repetition_penalty=1.0)),
            GenerateOptions(max_new_tokens=1),
            GenerateOptions(max_new_tokens=15, sampling=SamplingParams(temperature=1.1, top_p=1.0, seed=5,
                                                                       repetition_penalty=1.0))]
    # one more that looks back at its own tokens: its newest one is still on the device when the next is chosen
    prompts.append(torch.randint(0, cfg["vocab_size"], (7,), generator=g).tolist())
    opts.append(GenerateOptions(max_new_tokens=16, sampling=SamplingParams(temperature=0.9, top_p=0.95, seed=8,
                                                                           repetition_penalty=1.3,
                                                                           repetition_penalty_window=5)))
    results = {}
    for ahead in (False, True):
        rt = _runtime(d, "float32", block_size=4, num_blocks=num_blocks, max_batch_size=6, max_prefill_tokens=8)
        assert rt.look_ahead
        rt.look_ahead = ahead
        with_device_tokens, real_step = [], rt.engine.step
        rt.engine.step = lambda entries, **kw: (with_device_tokens.append(kw.get("device_tokens") is not None),
                                                real_step(entries, **kw))[1]
        seqs = [rt.submit(p, o) for p, o in zip(prompts, opts)]
        n_back = 0
        while not rt.scheduler.is_idle():
            n_back += len(rt.step().set_back)
        rt.run()
        assert all(s.error is None and s.pending == 0 for s in seqs)
        results[ahead] = [(list(s.generated_ids), s.finish_reason) for s in seqs]
        assert any(with_device_tokens) == ahead
        assert (n_back > 0) == (num_blocks == 13), f"{n_back} set back with {num_blocks} pages"
        rt.scheduler.reap(rt.engine.cache)
        rt.engine.cache.check()
        assert rt.engine.cache.free_pages() == num_blocks
    assert results[True] == results[False]
    assert results[True][1][0] == free_run[:free_run.index(eos)] and len(results[True][3][0]) == 1
    # the penalty changed what the last request drew (the test would not see a lost token otherwise), and its tokens
    # are the plain rule's over the plain model's logits
    import plain_llama as P
    from infernum_amd.sampling import token_uniform
    toks, sp = list(prompts[5]), opts[5].sampling
    differs = False
    for i, tok in enumerate(results[True][5][0]):
        logits = P.forward(cfg, w, toks)[-1]
        u = token_uniform(sp.seed, i)
        assert tok == P.sample_token(logits, sp.temperature, sp.top_p, u, sp.repetition_penalty, toks[-5:]), i
        differs = differs or tok != P.sample_token(logits, sp.temperature, sp.top_p, u, 1.0, [])
        toks.append(tok)
    assert differs


@pytest.mark.parametrize("seed", range(16))
def test_one_step_ahead_under_random_loads(folders, seed):
    """Random requests (greedy and sampled, some with a penalty on their last tokens, some with a stop token) over pools so small that requests are set
    back, with random limits of batch, portion and budget: in 32-bit, where a token's logits do not depend on what
    else is in its step, one step ahead and one step at a time give every request the same tokens and endings."""
    import random
    from infernum_amd import GenerateOptions, SamplingParams
    results = []
    for ahead in (False, True):
        rng = random.Random(1000 + seed)
        d, cfg, w = folders[rng.choice("AB")]
        vocab = cfg["vocab_size"]
        ps, n_req = rng.choice((2, 4, 8, 16)), rng.randint(2, 8)
        prompts = [[rng.randrange(vocab) for _ in range(rng.randint(1, 40))] for _ in range(n_req)]
        opts = []
        for _ in range(n_req):
            sp = None if rng.random() < 0.5 else SamplingParams(temperature=rng.choice((0.3, 0.7, 1.2)),
                                                               top_p=rng.choice((1.0, 0.9, 0.5)), seed=rng.randrange(1 << 30),
                                                               repetition_penalty=rng.choice((1.0, 1.2, 1.5)),
                                                               repetition_penalty_window=rng.choice((1, 3, 64)))
            opts.append(GenerateOptions(max_new_tokens=rng.randint(1, 24), sampling=sp,
                                        eos_token_id=rng.randrange(vocab) if rng.random() < 0.5 else None))
        longest = max(len(p) + o.max_new_tokens for p, o in zip(prompts, opts))
        pool = max(-(-longest // ps) + 1, rng.randint(3, 30))
        rt = _runtime(d, "float32", block_size=ps, num_blocks=pool, max_batch_size=rng.choice((2, 3, 5)),
                      max_prefill_tokens=rng.choice((3, 8, 64)), max_tokens_per_step=rng.choice((8, 16, 64)))
        assert rt.look_ahead
        rt.look_ahead = ahead
        seqs = [rt.submit(p, o) for p, o in zip(prompts, opts)]
        rt.run()
        assert all(s.pending == 0 for s in seqs)
        results.append([(list(s.generated_ids), s.error, s.finish_reason, len(s.generated_ids) <= o.max_new_tokens)
                        for s, o in zip(seqs, opts)])
        rt.engine.cache.check()
        assert rt.engine.cache.free_pages() == pool
    assert results[0] == results[1]

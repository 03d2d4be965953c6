"""The engine against the plain implementation on the GPU: whole requests, the tail
decoded one by one, portions of changing size, and mixed batches with so few pages
that they are used again; in 32-bit and in bfloat16."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_llama as P
import tiny_models as TM
import trace_tools as TT

pytestmark = pytest.mark.gpu

# Largest |difference| allowed, as a fraction of the RMS of the plain logits.
# fp32: sums of a few hundred to a few thousand fp32 products per element, a dozen
# such stages; measured ratios are 2e-6 to 4e-6, so 2e-5 holds a real fault out.
# bf16: every stored activation is rounded to 8 bits of mantissa (2^-9 relative);
# a dozen stages stacked, largest over ~10^5 elements.
TOL = {"float32": 2e-5, "bfloat16": 6e-2}
LENGTHS = {"A": (7, 40, 75, 33), "B": (5, 13, 29, 97, 64, 50), "C": (90, 41, 66, 120)}
MIXED_LENGTHS = {"A": (70, 131, 64, 190, 33, 97, 150, 66, 81, 120), "B": (129, 65, 200, 90, 47, 160, 72, 111, 99, 140),
                 "C": (90, 180, 66, 120, 75, 143, 35, 101, 170, 88)}
PAGE = {"A": 4, "B": 8, "C": 16}


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    out = {}
    for name in ("A", "B", "C"):
        for dt, tdt in (("float32", torch.float32), ("bfloat16", torch.bfloat16)):
            d = str(tmp_path_factory.mktemp(f"tiny{name}_{dt}"))
            TM.write_tiny(name, d, dtype=tdt)
            cfg, w = P.read_model(d)
            reqs = TT.make_requests(cfg["vocab_size"], LENGTHS[name], seed=11)
            ref = {r: P.forward(cfg, w, toks) for r, toks in reqs.items()}
            mreqs = TT.make_requests(cfg["vocab_size"], MIXED_LENGTHS[name], seed=23)
            mref = {r: P.forward(cfg, w, toks) for r, toks in mreqs.items()}
            out[(name, dt)] = (d, cfg, reqs, ref)
            out[(name, dt, "mixed")] = (d, cfg, mreqs, mref)
    return out


def _engine(model_dir, dtype, page_size, num_pages, poison=True, **kw):
    from infernum_amd import CacheConfig, Engine
    return Engine.from_pretrained(model_dir, dtype=dtype, **kw,
                                  cache_config=CacheConfig(page_size=page_size, num_pages=num_pages,
                                                           num_state_slots=8, poison_freed_pages=poison))


def _check(got, ref, dtype, what, every_place=True):
    worst, rms, where = TT.error_against(got, ref, every_place)
    print(f"{what}: max|diff| = {worst:.3e}, rms of logits = {rms:.3e}, ratio {worst / rms:.2e} at {where}")
    assert worst == worst, f"{what}: NaN in the logits at {where}"
    assert worst <= TOL[dtype] * rms, f"{what}: max|diff| {worst:.3e} > {TOL[dtype]} * rms {rms:.3e} at {where}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_whole(models, name, dtype):
    d, cfg, reqs, ref = models[(name, dtype)]
    eng = _engine(d, dtype, PAGE[name], 64)
    got = TT.run_steps(eng, TT.trace_whole(reqs))
    assert len(got) == sum(len(t) for t in reqs.values())
    _check(got, ref, dtype, f"{name} {dtype} whole")
    eng.cache.check()
    assert eng.cache.free_pages(0) == 64


def test_whole_with_the_hand_written_prefill_gemm(models):
    """Configuration B (width 128) with the many-row products on the hand-written LDS-tiled MFMA kernel where it
    takes the size (K in steps of 64: QKV, output projection, gate and up; the down projection's K of 352
    stays with the library): prompts of 97 and 64 tokens bring more than 64 rows."""
    import importlib
    L = importlib.import_module("infernum_amd.parts.linear")
    d, cfg, reqs, ref = models[("B", "bfloat16")]
    previous = L.set_prefill_gemm("mfma")
    try:
        eng = _engine(d, "bfloat16", PAGE["B"], 64)
        got = TT.run_steps(eng, TT.trace_whole(reqs))
    finally:
        L.set_prefill_gemm(previous)
    _check(got, ref, "bfloat16", "B bfloat16 whole, own prefill GEMM")
    # and the same logits as with the library's product: both accumulate in fp32 and round once
    lib = TT.run_steps(_engine(d, "bfloat16", PAGE["B"], 64), TT.trace_whole(reqs))
    worst, rms, where = TT.error_against(got, {r: torch.stack([lib[(r, i)] for i in range(len(t))]) for r, t in reqs.items()})
    assert worst <= 2e-2 * rms, f"own and library products differ by {worst:.3e} at {where}"


def test_steps_of_129_to_256_rows_through_the_tiled_kernel_with_k_split(models, monkeypatch):
    """Configuration B with its output projection (and, beyond what the table of the source holds, its QKV product)
    sent to the LDS-tiled kernel with K split in two for steps of 129 to 256 tokens: the norm and the rotary kernel
    add the partial sums.  Whole prompts of 129 to 200 tokens are such steps; the mixed trace has them beside
    smaller and larger ones.  Against the plain model, and the host library's program against the parts' calls."""
    import importlib
    L = importlib.import_module("infernum_amd.parts.linear")
    d, cfg, reqs, ref = models[("B", "bfloat16", "mixed")]
    H, nh, nkv = cfg["hidden_size"], cfg["num_attention_heads"], cfg["num_key_value_heads"]
    hd = H // nh
    monkeypatch.setitem(L.KNOWN_MID_ROWS, (H, nh * hd), ((129, 256, 2),))
    monkeypatch.setitem(L.KNOWN_MID_ROWS, ((nh + 2 * nkv) * hd, H), ((129, 160, 2), (161, 256, 1)))
    # and gate+up on the tiled kernel with the activation in its epilogue from 20 to 150 rows
    monkeypatch.setitem(L.KNOWN_GLU_ROWS, (2 * cfg["intermediate_size"], H), ((20, 150),))
    glu = L.plan(2 * cfg["intermediate_size"], H, torch.bfloat16, torch.bfloat16, "swiglu", False)
    assert {M: L.route_of(glu, M).kind for M in (19, 20, 150, 151)} == {19: "skinny", 20: "mfma_swiglu", 150: "mfma_swiglu", 151: "library"}
    kinds = {M: L.route_of(L.plan(H, nh * hd, torch.bfloat16, torch.bfloat16, None, True), M).kind for M in (128, 129, 256, 257)}
    assert kinds == {128: "skinny", 129: "mfma_split", 256: "mfma_split", 257: "library"}      # K of 128: one part up to 128 rows
    assert sum(129 <= len(t) <= 256 for t in reqs.values()) >= 4
    native = _engine(d, "bfloat16", PAGE["B"], 128)
    parts = _engine(d, "bfloat16", PAGE["B"], 128, executor="parts")
    assert "ia_gemm_mfma_split" in native.program.op_names and "ia_gemm_mfma_swiglu" in native.program.op_names
    a, b = TT.run_steps(native, TT.trace_whole(reqs)), TT.run_steps(parts, TT.trace_whole(reqs))
    _check(a, ref, "bfloat16", "B bfloat16 whole, 129 to 256 rows on the split tiled kernel")
    assert a.keys() == b.keys() and all(torch.equal(a[k], b[k]) for k in a)
    native.program.check_guards()
    prompt_len = {r: max(2, len(t) - 20) for r, t in reqs.items()}
    mixed, max_tokens = TT.trace_mixed(reqs, prompt_len, seed=5)
    eng = _engine(d, "bfloat16", PAGE["B"], max_tokens // PAGE["B"])
    _check(TT.run_steps(eng, mixed), ref, "bfloat16", "B bfloat16 mixed, split tiled kernel", every_place=False)
    eng.program.check_guards()


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_tail_one_by_one_rotation_inside_attention_or_before_it(models, name):
    """Steps of single tokens rotate queries and keys and write the pages inside the attention kernel; with the
    rotary kernel in front of it instead, every logit has the same bits."""
    import importlib
    A = importlib.import_module("infernum_amd.parts.attention")
    d, cfg, reqs, ref = models[(name, "bfloat16")]
    got = TT.run_steps(_engine(d, "bfloat16", PAGE[name], 64), TT.trace_tail_one_by_one(reqs, 32))
    previous = A.set_decode_rotation("separate")
    try:
        eng = _engine(d, "bfloat16", PAGE[name], 64)
        other = TT.run_steps(eng, TT.trace_tail_one_by_one(reqs, 32))
    finally:
        A.set_decode_rotation(previous)
    assert got.keys() == other.keys()
    for key in got:
        assert torch.equal(got[key], other[key]), key


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_tail_one_by_one(models, name, dtype):
    d, cfg, reqs, ref = models[(name, dtype)]
    eng = _engine(d, dtype, PAGE[name], 64)
    got = TT.run_steps(eng, TT.trace_tail_one_by_one(reqs, 32))
    _check(got, ref, dtype, f"{name} {dtype} tail one by one")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_portions(models, name, dtype):
    d, cfg, reqs, ref = models[(name, dtype)]
    eng = _engine(d, dtype, PAGE[name], 64)
    got = TT.run_steps(eng, TT.trace_portions(reqs))
    _check(got, ref, dtype, f"{name} {dtype} portions")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_mixed_with_page_reuse(models, name, dtype):
    d, cfg, reqs, ref = models[(name, dtype, "mixed")]
    prompt_len = {r: max(2, len(t) - 20) for r, t in reqs.items()}
    steps, max_tokens = TT.trace_mixed(reqs, prompt_len, seed=5)
    ps = PAGE[name]
    num_pages = max_tokens // ps
    total_pages = sum(-(-len(t) // ps) for t in reqs.values())
    assert total_pages > num_pages, "the pool must be too small to hold all requests without reuse"
    eng = _engine(d, dtype, ps, num_pages)
    got = TT.run_steps(eng, steps)
    _check(got, ref, dtype, f"{name} {dtype} mixed")
    eng.cache.check()
    assert eng.cache.free_pages(0) == num_pages


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sizes_that_no_fast_kernel_takes(tmp_path, dtype):
    """Head size 20, width 100, feed-forward width 150, vocabulary 333, pages of 5 tokens: every kernel either
    takes the size or hands over to a plain one; the logits are right all the same."""
    d = str(tmp_path / "D")
    TM.write_tiny("D", d, dtype={"float32": torch.float32, "bfloat16": torch.bfloat16}[dtype])
    cfg, w = P.read_model(d)
    reqs = TT.make_requests(cfg["vocab_size"], (23, 70, 9), seed=4)
    ref = {r: P.forward(cfg, w, toks) for r, toks in reqs.items()}
    for trace in (TT.trace_whole(reqs), TT.trace_portions(reqs), TT.trace_tail_one_by_one(reqs, 12)):
        got = TT.run_steps(_engine(d, dtype, 5, 40), trace)
        _check(got, ref, dtype, f"D {dtype}")


def test_cutting_does_not_change_fp32_logits(models):
    """In the 32-bit path a position's logits are the same bits however the tokens
    are cut into steps: each output is one chain of operations in a fixed order."""
    d, cfg, reqs, ref = models[("B", "float32")]
    a = TT.run_steps(_engine(d, "float32", 8, 64), TT.trace_whole(reqs))
    b = TT.run_steps(_engine(d, "float32", 8, 64), TT.trace_portions(reqs))
    c = TT.run_steps(_engine(d, "float32", 4, 128), TT.trace_tail_one_by_one(reqs))
    for k in a:
        assert torch.equal(a[k], b[k]), k
        assert torch.equal(a[k], c[k]), k


@pytest.mark.parametrize("name", ["B", "C"])
def test_plain_twins_of_the_fast_kernels_through_the_engine(models, name):
    """``kernels="generic"``: every matrix product and the attention on the plain kernels, also in bfloat16.
    Against the plain model, against the fast kernels (two sets of roundings of the same numbers), and in
    32-bit the very bits of the default path, which has no other kernels."""
    d, cfg, reqs, ref = models[(name, "bfloat16", "mixed")]
    prompt_len = {r: max(2, len(t) - 20) for r, t in reqs.items()}
    steps, max_tokens = TT.trace_mixed(reqs, prompt_len, seed=5)
    plain = _engine(d, "bfloat16", PAGE[name], max_tokens // PAGE[name], kernels="generic")
    assert not plain.model.blocks[0].mixer.use_mfma and plain.rt.kernels == "generic"
    got = TT.run_steps(plain, steps)
    _check(got, ref, "bfloat16", f"{name} bfloat16 mixed, plain kernels")
    fast = TT.run_steps(_engine(d, "bfloat16", PAGE[name], max_tokens // PAGE[name]), steps)
    worst, rms, where = TT.error_against(got, {r: torch.stack([fast[(r, i)] for i in range(len(t))])
                                               for r, t in reqs.items()})
    print(f"{name}: plain and fast kernels differ by {worst / rms:.2e} of the logits' RMS at {where}")
    assert worst <= 2 * TOL["bfloat16"] * rms
    d32, _, reqs32, _ = models[(name, "float32")]
    a = TT.run_steps(_engine(d32, "float32", PAGE[name], 64, kernels="generic"), TT.trace_portions(reqs32))
    b = TT.run_steps(_engine(d32, "float32", PAGE[name], 64), TT.trace_portions(reqs32))
    assert all(torch.equal(a[k], b[k]) for k in a)
    with pytest.raises(ValueError):
        _engine(d, "bfloat16", 8, 8, kernels="fastest")


@pytest.mark.parametrize("dtype,kernels", [("float32", "auto"), ("bfloat16", "generic")])
def test_trace_run_program(models, tmp_path, dtype, kernels):
    """bin/trace_run as a user starts it: steps on standard input, files out."""
    d, cfg, reqs, ref = models[("A", dtype)]
    prompt_len = {r: max(2, len(t) - 10) for r, t in reqs.items()}
    steps, max_tokens = TT.trace_mixed(reqs, prompt_len, seed=9)
    out = tmp_path / "out"
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    proc = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", d, "--dtype", dtype,
                           "--out", str(out), "--max-tokens", str(max_tokens), "--kernels", kernels],
                          input="".join(json.dumps(s) + "\n" for s in steps), text=True, capture_output=True,
                          timeout=600)
    assert proc.returncode == 0, proc.stderr[-3000:]
    assert proc.stdout.split("\n")[:-1] == [f"done {s['step']}" for s in steps]
    V = cfg["vocab_size"]
    pos, got = {}, {}
    for s in steps:
        n_want = sum(len(e["want"]) for e in s["entries"])
        arr = np.fromfile(out / f"{s['step']}.f32", dtype="<f4").reshape(n_want, V)
        row = 0
        for e in s["entries"]:
            base = pos.get(e["id"], 0)
            for w in e["want"]:
                got[(e["id"], base + w)] = torch.from_numpy(arr[row].copy())
                row += 1
            pos[e["id"]] = base + len(e["tokens"])
    _check(got, ref, dtype, f"trace_run A {dtype} mixed, kernels {kernels}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["B", "C"])
def test_recorded_decode_steps_equal_eager_ones(models, name, dtype):
    """Decode steps replayed from a HIP graph give the bits of the same steps launched one by one; every
    replay is checked, with eager steps (portions of prompts) and synchronisations between them."""
    from infernum_amd import CacheConfig, Engine, StepEntry
    d, cfg, reqs, ref = models[(name, dtype, "mixed")]
    eager = Engine.from_pretrained(d, dtype=dtype, use_graphs=False,
                                   cache_config=CacheConfig(page_size=PAGE[name], num_pages=128, num_state_slots=8))
    graphed = Engine.from_pretrained(d, dtype=dtype, use_graphs=True,
                                     cache_config=CacheConfig(page_size=PAGE[name], num_pages=128, num_state_slots=8))
    assert graphed.use_graphs and not eager.use_graphs
    names = sorted(reqs, key=lambda r: -len(reqs[r]))[:3]      # the three longest: 41 + 40 tokens at least
    fed = {r: 0 for r in names}
    for r in names:                                   # prompts in one step each
        n = 20 + 7 * names.index(r)
        for eng in (eager, graphed):
            eng.step([StepEntry(r, reqs[r][:n], [])])
        fed[r] = n
    for it in range(40):
        live = names if it % 7 else names[:2]         # the batch size changes now and then: another shape
        entries = [StepEntry(r, reqs[r][fed[r]:fed[r] + 1], [0]) for r in live]
        a, b = eager.step(entries), graphed.step(entries)
        torch.cuda.synchronize()
        assert torch.equal(a, b), it
        for r in live:
            fed[r] += 1
        if it % 9 == 4:                               # an eager step of another kind between replays
            for eng in (eager, graphed):
                eng.step([StepEntry("x", reqs[names[0]][:11], [10])])
                eng.end("x")
    assert graphed.graph_replays >= 30
    got = {(r, fed[r] - 1): graphed.step([StepEntry(r, reqs[r][fed[r]:fed[r] + 1], [0])])[0].cpu() for r in names[:1]}
    _check({(names[0], fed[names[0]]): got[(names[0], fed[names[0]] - 1)]}, ref, dtype, f"{name} {dtype} recorded decode",
           every_place=False)


def test_time_per_kernel_switch(models):
    """INFERNUM_PROFILE=1 / set_profile: every kernel call is timed on the device and summed by function; an
    engine made meanwhile records no graphs; the logits are those of an engine without it."""
    from infernum_amd.kernels import api as K
    d, cfg, reqs, ref = models[("B", "bfloat16")]
    plain = TT.run_steps(_engine(d, "bfloat16", 8, 64), TT.trace_tail_one_by_one(reqs, 8))
    before = K.set_profile(True)
    try:
        K.profile_report(reset=True)
        eng = _engine(d, "bfloat16", 8, 64)
        assert not eng.use_graphs
        timed = TT.run_steps(eng, TT.trace_tail_one_by_one(reqs, 8))
        rep = K.profile_report(reset=True)
    finally:
        K.set_profile(before)
    assert all(torch.equal(plain[k], timed[k]) for k in plain)
    steps = len(TT.trace_tail_one_by_one(reqs, 8))
    layers = cfg["num_hidden_layers"]
    assert rep["embed"][0] == steps and rep["add_rmsnorm"][0] == steps * (2 * layers + 1)
    assert {"attention_decode_rotating", "attention_prefill", "gemm_skinny", "rope_kv_append"} <= set(rep)
    assert all(calls > 0 and ms > 0 for calls, ms in rep.values())
    assert K.profile_report() == {}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_native_program_makes_the_launches_of_the_parts(models, name, dtype):
    """A step run by the host library from one call (the default where every part has a native description)
    gives the bits of the same step run by the parts' own forward, launch by launch from Python: whole prompts,
    portions, single tokens (rotation inside the attention kernel), mixed steps, with pages used again."""
    d, cfg, reqs, ref = models[(name, dtype, "mixed")]
    prompt_len = {r: max(2, len(t) - 20) for r, t in reqs.items()}
    mixed, max_tokens = TT.trace_mixed(reqs, prompt_len, seed=5)
    traces = (TT.trace_whole(reqs), TT.trace_portions(reqs), mixed)
    native = _engine(d, dtype, PAGE[name], max_tokens // PAGE[name])
    parts = _engine(d, dtype, PAGE[name], max_tokens // PAGE[name], executor="parts")
    assert native.program is not None and parts.program is None
    assert native.program.num_ops >= 9 * cfg["num_hidden_layers"]      # norm, product, rotation, attention, product; norm, two products (three with the activation)
    assert native.program.num_python_ops == 0                              # nothing of a Llama step is a call into Python
    for steps in traces:
        a, b = TT.run_steps(native, steps), TT.run_steps(parts, steps)
        assert a.keys() == b.keys()
        for k in a:
            assert torch.equal(a[k], b[k]), k
        native.program.check_guards()              # no launch wrote past the end of its intermediate
    for kernels in ("generic",):
        a = TT.run_steps(_engine(d, dtype, PAGE[name], 64, kernels=kernels), TT.trace_portions(reqs))
        b = TT.run_steps(_engine(d, dtype, PAGE[name], 64, kernels=kernels, executor="parts"), TT.trace_portions(reqs))
        assert all(torch.equal(a[k], b[k]) for k in a)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("limit", [7, 64, 129, 300])
def test_intermediates_of_the_program_are_large_enough_for_steps_of_every_shape(models, dtype, limit):
    """An engine whose steps take at most ``limit`` tokens has intermediates for exactly that many: steps that fill
    the limit (one long portion; single tokens only; both) leave the guards behind every intermediate untouched and
    give the bits of the parts' own forward."""
    from infernum_amd import CacheConfig, Engine, StepEntry
    d, cfg, reqs, ref = models[("C", dtype, "mixed")]
    V = cfg["vocab_size"]
    engines = [Engine.from_pretrained(d, dtype=dtype, max_tokens_per_step=limit, executor=ex, use_graphs=False,
                                      cache_config=CacheConfig(page_size=8, num_pages=limit + 40, num_state_slots=limit + 2))
               for ex in ("native", "parts")]
    g = torch.Generator().manual_seed(limit)
    toks = lambda n: torch.randint(0, V, (n,), generator=g).tolist()
    singles = min(limit, 90)
    steps = [[StepEntry("long", toks(limit), [0, limit - 1])],
             [StepEntry(("s", i), toks(1), [0]) for i in range(singles)],
             [StepEntry(("s", i), toks(1), [0]) for i in range(singles)]]
    if limit > 3:
        half = limit // 2
        steps.append([StepEntry(("s", i), toks(1), [0]) for i in range(min(half, singles))] +
                     [StepEntry("other", toks(limit - min(half, singles)), [])])
    outs = []
    for eng in engines:
        res = []
        for entries in steps:
            res.append(eng.step(entries).cpu())
            if entries[0].request == "long":
                eng.end("long")
        outs.append(res)
    engines[0].program.check_guards()
    for a, b in zip(*outs):
        assert torch.equal(a, b)
    with pytest.raises(Exception):
        engines[0].step([StepEntry("too long", toks(limit + 1), [])])

"""The engine against the plain implementation at the lengths that the benchmarks time: prompts of 2,304 and
8,200 tokens whole, in portions of 2,048 and with their last 32 tokens one by one; a dozen decoded tokens after
33,000 tokens of context; loud keys late in a prompt of 8,200 tokens.

Short tests cannot show what these lengths have: the prompt kernel's launch shapes (four heads a workgroup with
rows from both ends of the request, four heads with rows as they come, two heads), dozens of tiles of keys per
row with a reference point of the exponentials that moves late, workgroups that queue for the compute units,
block tables longer than the slice the decode kernel keeps in LDS, keys split over dozens of workgroups.
The plain model runs in float64 with its attention a head and a block of rows at a time
(``plain_llama.causal_attention_blocked``, held to the loop over tokens by ``test_plain_pins``).  One folder
per configuration, stored in bfloat16, serves both types, as in ``test_gpu_real_sizes``.
"""
import math

import pytest
import torch

import plain_llama as P
import tiny_models as TM
import trace_tools as TT
from part_harness import build, rel_err, runtime

pytestmark = pytest.mark.gpu
TOL = {"float32": 2e-5, "bfloat16": 6e-2}
LONG, SHORT = 8200, 2304

# A, B (one key/value head, llama3 scaling) and C (a window of 24 on two layers of three) as everywhere; W: C's
# sizes with a window of 1,500, which spans two dozen tiles and ends inside one; E: sixteen heads over four of
# 128, the head size and grouping at which the prompt kernel puts four heads into a workgroup.
RAW = {
    "A": dict(TM.TINY_A, max_position_embeddings=65536),
    "B": dict(TM.TINY_B, max_position_embeddings=65536),
    "C": dict(TM.TINY_C, max_position_embeddings=65536),
    "W": dict(TM.TINY_C, max_position_embeddings=65536, sliding_window=1500),
    "E": dict(model_type="llama", num_hidden_layers=2, hidden_size=192, num_attention_heads=16,
              num_key_value_heads=4, head_dim=128, intermediate_size=328, vocab_size=300, rope_theta=500000.0,
              rms_norm_eps=1e-5, tie_word_embeddings=False, max_position_embeddings=65536),
}
KW = dict(TM.SPEC_KW, W=TM.SPEC_KW["C"], E=TM.SPEC_KW["B"])
_made = {}


def _model(name, tmp_path_factory):
    """(folder, plain config, plain weights, the request's tokens, float64 logits of the whole request)."""
    if name not in _made:
        from infernum_amd.config import LlamaConfig
        from infernum_amd.weights import write_random_model
        d = str(tmp_path_factory.mktemp("lengths_" + name))
        write_random_model(LlamaConfig.from_dict(RAW[name], where="lengths " + name), d, 40 + len(_made),
                           dtype=torch.bfloat16, **KW[name])
        cfg, w = P.read_model(d)
        toks = TT.make_requests(cfg["vocab_size"], (LONG,), seed=17)["r0"]
        torch.set_num_threads(16)
        _made[name] = (d, cfg, w, toks, P.forward(cfg, w, toks, blocked=True))
    return _made[name]


def _engine(d, dtype, pages, ps=16, tokens_per_step=LONG + 56):
    from infernum_amd import CacheConfig, Engine
    return Engine.from_pretrained(d, dtype=dtype, max_tokens_per_step=tokens_per_step, cache_config=CacheConfig(
        page_size=ps, num_pages=pages, num_state_slots=4, poison_freed_pages=True))


def _portions(toks, size):
    steps, p = [], 0
    while p < len(toks):
        n = min(size, len(toks) - p)
        last = p + n == len(toks)
        steps.append({"step": len(steps), "entries": [{"id": "r", "tokens": toks[p:p + n], "want": list(range(n))}],
                      "end": ["r"] if last else []})
        p += n
    return steps


@pytest.fixture
def launch_shapes(monkeypatch):
    """The launch shapes that the prompt kernel was given meanwhile (both executors ask kernels.api for them)."""
    from infernum_amd.kernels import api
    seen = []
    real = api.prefill_launch_shape

    def spy(*a, **kw):
        shape = real(*a, **kw)
        seen.append(shape)
        return shape
    monkeypatch.setattr(api, "prefill_launch_shape", spy)
    return seen


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(RAW))
def test_long_prompts_whole_in_portions_and_with_a_decoded_tail(name, dtype, tmp_path_factory, launch_shapes):
    d, cfg, w, toks, ref = _model(name, tmp_path_factory)
    eng = _engine(d, dtype, pages=(LONG + 63) // 64 * 4)
    lengths = (SHORT, 4096, LONG) if name == "E" else (SHORT, LONG)
    for n in lengths:
        reqs, want = {"r": toks[:n]}, {"r": ref[:n]}          # a prefix's logits are the whole request's: causal
        for way, steps in (("whole", TT.trace_whole(reqs)), ("portions of 2,048", _portions(toks[:n], 2048)),
                           ("last 32 one by one", TT.trace_tail_one_by_one(reqs, 32))):
            if way == "last 32 one by one" and n == 4096:
                continue
            got = TT.run_steps(eng, steps)
            worst, rms, where = TT.error_against(got, want)
            line = f"{name} {dtype} {n} tokens {way}: {worst / rms:.2e} of the logits' RMS at {where}"
            assert worst == worst and worst <= TOL[dtype] * rms, line
            print(line)
    eng.cache.check()
    eng.program.check_guards()
    assert all(g.allocator.num_free == g.allocator.num_pages for g in eng.cache.groups)
    if name == "E" and dtype == "bfloat16":
        from infernum_amd.kernels import api
        assert torch.cuda.get_device_properties(0).multi_processor_count == 256, "the lengths are chosen for 256 compute units"
        assert {4 | api.PREFILL_PAIRED, 4, 2 | api.PREFILL_PAIRED, 2} <= set(launch_shapes), sorted(set(launch_shapes))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "W"])
def test_a_dozen_tokens_decoded_after_33000(name, dtype, tmp_path_factory):
    """Pages of 16 tokens: 2,064 entries in a block table, more than the decode kernel keeps in LDS; the keys of
    the one request are split over dozens of workgroups.  W: the window group has long given back the pages of
    the first 31,000 tokens.  The plain model works out its last layer at
    the twelve places only."""
    from infernum_amd.engine import StepEntry
    from infernum_amd.kernels import api
    d, cfg, w, _, _ = _model(name, tmp_path_factory)
    n_ctx, n_new = 33000, 12
    toks = TT.make_requests(cfg["vocab_size"], (n_ctx + n_new,), seed=23)["r0"]
    torch.set_num_threads(16)
    ref = P.forward(cfg, w, toks, blocked=True, rows=range(n_ctx, n_ctx + n_new))
    pages = (n_ctx + n_new) // 16 + 2
    eng = _engine(d, dtype, pages=pages, tokens_per_step=8192)
    for p in range(0, n_ctx, 8192):
        eng.step([StepEntry("r", toks[p:min(n_ctx, p + 8192)], [])])
    assert api.decode_splits(1, cfg["num_attention_heads"], cfg["num_key_value_heads"], n_ctx) >= 4
    rms = ref.pow(2).mean().sqrt().item()
    worst = 0.0
    for i in range(n_new):
        row = eng.step([StepEntry("r", [toks[n_ctx + i]], [0])])[0].double().cpu()
        worst = max(worst, (row - ref[i]).abs().max().item())
    print(f"{name} {dtype} decoding after {n_ctx} tokens: {worst / rms:.2e} of the logits' RMS")
    assert worst == worst and worst <= TOL[dtype] * rms
    if name == "W":
        window = [g for g in eng.cache.groups if g.kind == "window"][0]
        assert window.allocator.num_pages - window.allocator.num_free <= 1500 // 16 + 3
    eng.end("r")
    eng.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_loud_keys_late_in_a_prompt_of_8200(dtype):
    """The attention part alone, eight heads over two of 128, with weights that let the input rows set the
    scores: every query has a lifted first component, key 5,000 answers it with 2^29 times the weight of all
    before it and key 7,000 with 2^58 times that.  Every later row's reference point of the exponentials moves
    after 78 and after 109 tiles of keys; a kernel that scales its sums wrongly then, or that keeps stale
    exponentials, returns something other than the loud key's values."""
    from test_gpu_parts import _run_attention
    nh, nkv, d = 8, 2, 128
    H, T = 3 * d, LONG
    rt = runtime(dtype)
    eye = torch.eye(H)
    w = {"q_proj.weight": torch.cat([eye[:d]] * nh), "k_proj.weight": torch.cat([eye[d:2 * d]] * nkv),
         "v_proj.weight": torch.cat([eye[2 * d:]] * nkv), "o_proj.weight": torch.eye(H, nh * d)}
    att, wd = build("mixer", "attention", {"hidden_size": H, "num_heads": nh, "num_kv_heads": nkv, "head_dim": d,
                                           "position": {"kind": "none", "params": {}}}, rt, tensors=w)
    g = torch.Generator().manual_seed(8)
    x = torch.randn(T, H, generator=g) * 0.5
    scale = 1.0 / math.sqrt(d)
    x[:, 0] += 4.0                                     # every query's first component
    x[5000, d] = 20.0 / (4.0 * scale)
    x[7000, d] = 60.0 / (4.0 * scale)
    x = x.to(torch.bfloat16).float()
    torch.set_num_threads(16)
    q = x[:, :d].double().reshape(T, 1, d).expand(T, nh, d).contiguous()
    k = x[:, d:2 * d].double().reshape(T, 1, d).expand(T, nkv, d).contiguous()
    v = x[:, 2 * d:].double().reshape(T, 1, d).expand(T, nkv, d).contiguous()
    want = P.causal_attention_blocked(q, k, v, scale).reshape(T, nh * d)[:, :H]
    assert (want[6999, :d] - x[5000, 2 * d:].double()).abs().max() < 1e-3       # the plain result follows the loud keys
    assert (want[8199, :d] - x[7000, 2 * d:].double()).abs().max() < 1e-3
    assert (want[4999, :d] - x[5000, 2 * d:].double()).abs().max() > 0.1
    for cuts in ([T], [4096, T - 4096], [2048] * 4 + [T - 8192], [T - 32] + [1] * 32):
        got = _run_attention(att, rt, x, cuts, 16, window_pages=T // 16 + 2)
        err = rel_err(got, want)
        print(f"loud keys {dtype} cuts {cuts[:5]}: {err:.2e}")
        assert err <= (2e-5 if dtype == "float32" else 3e-2), cuts

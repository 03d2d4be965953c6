"""The engine against the plain implementation at the layer sizes of Llama-3.1-8B (width 4,096, 32 heads on 8
key/value heads of 128, feed-forward width 14,336, the vocabulary of 128,256; two layers), and of the 13B, 1B and
70B shapes that the benchmarks also run, under all four ways of cutting, in 32-bit and in bfloat16.

The tiny configurations cannot show what only these sizes have: inner dimensions of 4,096 and 14,336 split over
workgroups and joined by the next kernel, four heads of 128 to a workgroup, a head of 128,256 rows.  Their
tolerances do not carry over either (rounding grows with the sizes), so the tolerances here come from the
plain implementation itself:

* 32-bit: the plain model in fp32 differs from the plain model in float64 by E32 (sums of thousands of fp32
  products); the engine's 32-bit path may differ from float64 by twice that.
* bfloat16: the plain model with every stored activation rounded to bfloat16 (``round_to``) differs from the
  exact one by Ebf; that is what rounding alone does at these sizes.  The engine may differ from the exact
  model by one and a half times that, and from the rounding model too (two sets of roundings, independent of each other).
  The largest difference over millions of logits is a loose measure (one unlucky logit sets it), so the root mean
  square of the difference is held as well, and tightly: the engine rounds where the rounding model rounds, so its
  root-mean-square distance from the exact model may be 1.1 times the rounding model's (measured: 0.84 to 1.0
  times), and its distance from the rounding model 1.2 times that (two sets of roundings of the same numbers,
  partly the same ones: measured 0.6 to 1.03 times, where independent sets would give the square root of two).
  A defect of three per cent in one bfloat16 kernel at these sizes adds some 3e-2 to distances of 1e-2.
"""
import pytest
import torch

import plain_llama as P
import trace_tools as TT

pytestmark = pytest.mark.gpu

_LLAMA3 = {"rope_type": "llama3", "low_freq_factor": 1.0, "high_freq_factor": 4.0, "original_max_position_embeddings": 8192}
# Two layers of each shape that the benchmarks run.  "13b": as many key/value heads as heads (one query head a
# workgroup in the attention kernels, one used column of sixteen in the decode kernel's tiles), widths 5,120 and
# 13,824 (54 chunks of 256 for the split products), no scaling of the rotation.  "1b": heads of 64, the head tied to
# the embedding, a scaling factor of 32; its vocabulary is cut to 16,001 (odd) to keep the float64 model short.
SHAPES = {
    "8b": {"model_type": "llama", "vocab_size": 128256, "hidden_size": 4096, "intermediate_size": 14336,
           "num_hidden_layers": 2, "num_attention_heads": 32, "num_key_value_heads": 8, "rope_theta": 500000.0,
           "max_position_embeddings": 8192, "rms_norm_eps": 1e-5, "rope_scaling": dict(_LLAMA3, factor=8.0)},
    "13b": {"model_type": "llama", "vocab_size": 32000, "hidden_size": 5120, "intermediate_size": 13824,
            "num_hidden_layers": 2, "num_attention_heads": 40, "num_key_value_heads": 40, "rope_theta": 10000.0,
            "max_position_embeddings": 4096, "rms_norm_eps": 1e-5},
    "1b": {"model_type": "llama", "vocab_size": 16001, "hidden_size": 2048, "intermediate_size": 8192,
           "num_hidden_layers": 2, "num_attention_heads": 32, "num_key_value_heads": 8, "head_dim": 64,
           "rope_theta": 500000.0, "max_position_embeddings": 131072, "rms_norm_eps": 1e-5,
           "tie_word_embeddings": True, "rope_scaling": dict(_LLAMA3, factor=32.0)},
    # one layer of the 70B shape: widths 8,192 and 28,672 (112 chunks of 256 in the down projection), eight query heads
    # to a key/value head, products whose rows go to the library from 17 on by the table; a short vocabulary again
    "70b": {"model_type": "llama", "vocab_size": 16001, "hidden_size": 8192, "intermediate_size": 28672,
            "num_hidden_layers": 1, "num_attention_heads": 64, "num_key_value_heads": 8, "rope_theta": 500000.0,
            "max_position_embeddings": 131072, "rms_norm_eps": 1e-5, "rope_scaling": dict(_LLAMA3, factor=8.0)},
}
LENGTHS = (300, 61, 130)


def _ratio(a: torch.Tensor, ref: torch.Tensor) -> float:
    return float((a.double() - ref).abs().max() / ref.pow(2).mean().sqrt())


@pytest.fixture(scope="module", params=list(SHAPES))
def real(request, tmp_path_factory):
    RAW = SHAPES[request.param]
    from infernum_amd.config import LlamaConfig
    from infernum_amd.weights import write_random_model
    d = str(tmp_path_factory.mktemp("real_sizes_" + request.param))
    cfg = LlamaConfig.from_dict(RAW, where="real sizes " + request.param)
    write_random_model(cfg, d, 5, dtype=torch.bfloat16, made_on="cuda:0", norm_init=("uniform", 0.5, 1.5))
    pcfg, w = P.read_model(d)
    reqs = TT.make_requests(RAW["vocab_size"], LENGTHS, seed=1)
    torch.set_num_threads(16)
    w64 = {k: v.double() for k, v in w.items()}
    exact = {r: P.forward(pcfg, w64, t) for r, t in reqs.items()}
    rounding = {r: P.forward(pcfg, w64, t, round_to=torch.bfloat16) for r, t in reqs.items()}
    del w64
    short = min(reqs, key=lambda r: len(reqs[r]))
    e32 = _ratio(P.forward(pcfg, w, reqs[short], dtype=torch.float32), exact[short])
    ebf = max(_ratio(rounding[r], exact[r]) for r in reqs)
    # the same in the root mean square over all logits: what the rows are like, where the largest difference is
    # set by one unlucky logit among millions
    sq = sum(float((rounding[r] - exact[r]).pow(2).sum()) for r in reqs)
    ebf_rms = (sq / sum(float(exact[r].pow(2).sum()) for r in reqs)) ** 0.5
    print(f"real sizes {request.param}: plain fp32 against float64 {e32:.2e}; plain with bfloat16 roundings against exact "
          f"{ebf:.2e} at the worst logit, {ebf_rms:.2e} in the root mean square")
    assert 1e-6 < e32 < 1e-4 and 1e-2 < ebf < 0.3, "the plain implementations disagree in a way rounding does not explain"
    return d, reqs, exact, rounding, e32, ebf, ebf_rms


def _traces(reqs):
    prompt_len = {r: len(t) - 24 for r, t in reqs.items()}
    mixed, max_tokens = TT.trace_mixed(reqs, prompt_len, seed=3, max_live=3)
    return max_tokens, (("whole", TT.trace_whole(reqs)), ("tail", TT.trace_tail_one_by_one(reqs, 32)),
                        ("portions", TT.trace_portions(reqs)), ("mixed", mixed))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_all_ways_of_cutting_at_real_sizes(real, dtype):
    from infernum_amd import CacheConfig, Engine
    d, reqs, exact, rounding, e32, ebf, ebf_rms = real
    max_tokens, traces = _traces(reqs)
    eng = Engine.from_pretrained(d, dtype=dtype, cache_config=CacheConfig(
        page_size=16, num_pages=max_tokens // 16 + 1, num_state_slots=4, poison_freed_pages=True))
    tol = 2 * e32 if dtype == "float32" else 1.5 * ebf
    for name, steps in traces:
        got = TT.run_steps(eng, steps)
        worst, rms, where = TT.error_against(got, exact)
        line = f"real sizes {dtype} {name}: {worst / rms:.2e} of the logits' RMS at {where} (allowed {tol:.2e})"
        assert worst == worst, f"{name}: NaN at {where}"
        assert worst <= tol * rms, line
        if dtype == "bfloat16":
            worst_r, rms_r, where_r = TT.error_against(got, rounding)
            line += f"; against the rounding plain model {worst_r / rms_r:.2e}"
            assert worst_r <= tol * rms_r, line
            to_exact, to_rounding = TT.rms_error_against(got, exact), TT.rms_error_against(got, rounding)
            line += (f"; root mean square: {to_exact:.2e} from the exact model, {to_rounding:.2e} from the rounding one "
                     f"(which is {ebf_rms:.2e} from the exact one)")
            assert to_exact <= 1.1 * ebf_rms and to_rounding <= 1.2 * ebf_rms, line
        print(line)
    eng.cache.check()
    eng.program.check_guards()
    assert all(g.allocator.num_free == g.allocator.num_pages for g in eng.cache.groups)

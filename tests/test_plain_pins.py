"""Pins of the plain implementation: what fixes each formula beside the
reference's text.  Each test is chosen so that a plausible mistake fails it."""
import math

import torch

import plain_llama as P

torch.manual_seed(0)


def test_rmsnorm_reference_vector():
    # infernum-cuda/src/inner/cuda/ops/rmsnorm.rs:171-203: [1,2,3,4], w = 1 -> x / sqrt(7.5)
    x = torch.tensor([[1.0, 2.0, 3.0, 4.0]], dtype=torch.float64)
    out = P.rms_norm(x, torch.ones(4, dtype=torch.float64), 1e-6)
    assert torch.allclose(out, x / math.sqrt(7.5), atol=1e-6)


def test_rmsnorm_eps_inside_root_and_weight_multiplies():
    x = torch.zeros(1, 8, dtype=torch.float64)
    x[0, 0] = 1e-4                      # mean(x^2) = 1.25e-9, far below eps
    w = torch.full((8,), 2.0, dtype=torch.float64)
    out = P.rms_norm(x, w, 1e-6)
    assert abs(out[0, 0].item() - 1e-4 / math.sqrt(1.25e-9 + 1e-6) * 2.0) < 1e-12
    # a (1 + w) convention or eps outside the root gives other numbers
    assert abs(out[0, 0].item() - 1e-4 / (math.sqrt(1.25e-9) + 1e-6) * 2.0) > 1e-3


def test_rmsnorm_equals_library_and_scale_invariance():
    x = torch.randn(5, 96, dtype=torch.float64)
    w = torch.rand(96, dtype=torch.float64) + 0.5
    lib = torch.nn.functional.rms_norm(x, (96,), w, eps=1e-5)
    assert torch.allclose(P.rms_norm(x, w, 1e-5), lib, atol=1e-12)
    assert torch.allclose(P.rms_norm(3.0 * x, w, 1e-30), P.rms_norm(x, w, 1e-30), atol=1e-12)


def test_rope_reference_vector_half_split():
    # infernum-cuda/src/inner/cuda/ops/rope.rs:835-885: [a,b,c,d], pos 1, theta 1e4, d = 4
    a, b, c, d = 1.0, 2.0, 3.0, 4.0
    f = P.rope_frequencies(4, 10000.0, None)
    assert torch.allclose(f, torch.tensor([1.0, 0.01], dtype=torch.float64))
    x = torch.tensor([[[a, b, c, d]]], dtype=torch.float64)
    out = P.rope(x, torch.tensor([1]), f)[0, 0]
    c0, s0, c1, s1 = math.cos(1.0), math.sin(1.0), math.cos(0.01), math.sin(0.01)
    want = torch.tensor([a * c0 - c * s0, b * c1 - d * s1, c * c0 + a * s0, d * c1 + b * s1], dtype=torch.float64)
    assert torch.allclose(out, want, atol=1e-12)
    # the interleaved pairing would give something else (rope.rs:1275)
    inter = torch.tensor([a * c0 - b * s0, a * s0 + b * c0, c * c1 - d * s1, c * s1 + d * c1], dtype=torch.float64)
    assert not torch.allclose(out, inter, atol=1e-3)


def test_rope_identity_at_zero_and_norm():
    # rope.rs:804-832
    x = torch.randn(3, 2, 16, dtype=torch.float64)
    f = P.rope_frequencies(16, 10000.0, None)
    assert torch.allclose(P.rope(x, torch.zeros(3, dtype=torch.long), f), x)
    y = P.rope(x, torch.tensor([5, 17, 300]), f)
    assert torch.allclose(y.norm(dim=-1), x.norm(dim=-1), atol=1e-12)


def test_rope_scores_depend_on_distance_only():
    f = P.rope_frequencies(32, 500000.0, None)
    q = torch.randn(1, 1, 32, dtype=torch.float64)
    k = torch.randn(1, 1, 32, dtype=torch.float64)
    def score(pq, pk):
        return (P.rope(q, torch.tensor([pq]), f) * P.rope(k, torch.tensor([pk]), f)).sum().item()
    assert abs(score(10, 3) - score(110, 103)) < 1e-10
    assert abs(score(10, 3) - score(3, 10)) > 1e-6        # a wrong sign of the angle swaps these


def test_llama3_scaling_three_bands():
    sc = dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
              original_max_position_embeddings=64)
    base = P.rope_frequencies(32, 500000.0, None)
    scaled = P.rope_frequencies(32, 500000.0, sc)
    wl = 2 * math.pi / base
    # wavelengths 6.3, 14.3 < 16: unchanged; 32.4: blended; >= 73 > 64: divided by 8
    assert torch.allclose(scaled[:2], base[:2])
    assert base[2] / 8 < scaled[2] < base[2]
    r = (64 / wl[2] - 1.0) / 3.0
    assert torch.allclose(scaled[2], (1 - r) * base[2] / 8 + r * base[2])
    assert torch.allclose(scaled[3:], base[3:] / 8)
    one = dict(sc, factor=1.0)
    assert torch.allclose(P.rope_frequencies(32, 500000.0, one), base)      # rope.rs:982 in spirit


def test_llama3_scaling_blends_in_the_frequency_between_the_bands_edges():
    """Between the edges the scaled frequency over the unscaled one is affine in the frequency itself, from 1/factor
    at the edge of the long waves (f = 2 pi low / n) to 1 at the edge of the short ones (f = 2 pi high / n):
    the reference's ramp (infernum/src/rope.rs:104-110) is (n / wavelength - low) / (high - low), and n / wavelength
    is n f / (2 pi).  A blend that is affine in the wavelength, or in the index of the pair, fails this; so do
    swapped edges."""
    n, low, high, factor = 8192, 1.0, 4.0, 8.0
    sc = dict(rope_type="llama3", factor=factor, low_freq_factor=low, high_freq_factor=high,
              original_max_position_embeddings=n)
    base = P.rope_frequencies(2048, 500000.0, None)           # many pairs, so that dozens fall between the edges
    scaled = P.rope_frequencies(2048, 500000.0, sc)
    f_long, f_short = 2 * math.pi * low / n, 2 * math.pi * high / n
    inside = (base > f_long) & (base < f_short)
    assert int(inside.sum()) >= 40
    ratio = scaled[inside] / base[inside]
    want = 1 / factor + (1 - 1 / factor) * (base[inside] - f_long) / (f_short - f_long)
    assert torch.allclose(ratio, want, rtol=1e-12, atol=0)
    assert torch.all(ratio[:-1] > ratio[1:])                    # pairs of rising index have falling frequencies
    # and it is not affine in the wavelength: the middle of the band in wavelength is not its middle in the ratio
    wl = 2 * math.pi / base[inside]
    mid = torch.argmin((wl - (n / low + n / high) / 2).abs())
    assert abs(float(ratio[mid]) - (1 / factor + 1) / 2) > 0.1


def _sdpa(q, k, v, scale):
    # library attention on [heads, T, d]
    return torch.nn.functional.scaled_dot_product_attention(
        q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1), is_causal=True, scale=scale).transpose(0, 1)


def test_attention_equals_library_when_heads_equal():
    T, nh, d = 9, 3, 8
    q, k, v = (torch.randn(T, nh, d, dtype=torch.float64) for _ in range(3))
    out = P.causal_attention(q, k, v, 0.3)
    assert torch.allclose(out, _sdpa(q, k, v, 0.3), atol=1e-12)
    assert torch.allclose(out[0], v[0])                     # the first query sees one key


def test_attention_grouping_equals_repeated_heads():
    T, nh, nkv, d = 7, 6, 2, 4
    q = torch.randn(T, nh, d, dtype=torch.float64)
    k, v = (torch.randn(T, nkv, d, dtype=torch.float64) for _ in range(2))
    out = P.causal_attention(q, k, v, 0.5)
    rk, rv = k.repeat_interleave(nh // nkv, dim=1), v.repeat_interleave(nh // nkv, dim=1)
    assert torch.allclose(out, _sdpa(q, rk, rv, 0.5), atol=1e-12)
    # a wrong mapping (h % nkv) differs
    wk, wv = k.repeat(1, nh // nkv, 1), v.repeat(1, nh // nkv, 1)
    assert not torch.allclose(out, _sdpa(q, wk, wv, 0.5), atol=1e-3)


def test_attention_window():
    T, d, w = 12, 4, 5
    q, k, v = (torch.randn(T, 1, d, dtype=torch.float64) for _ in range(3))
    out = P.causal_attention(q, k, v, 1.0, window=w)
    full = P.causal_attention(q, k, v, 1.0)
    assert torch.allclose(out[:w], full[:w])                # the window has not filled yet
    t = 9
    s = (k[t - w + 1:t + 1, 0] @ q[t, 0])
    want = torch.softmax(s, 0) @ v[t - w + 1:t + 1, 0]
    assert torch.allclose(out[t, 0], want, atol=1e-12)
    assert not torch.allclose(out[t], full[t], atol=1e-6)


def test_blocked_attention_is_the_attention_row_by_row():
    """The form for long sequences (a head and a block of rows at a time) against the loop over tokens: whole,
    under a window that cuts inside a block, with rounded exponentials, and for a few places only."""
    q, k, v = (torch.randn(75, n, 8, dtype=torch.float64) for n in (6, 2, 2))
    for window in (None, 9, 40):
        for round_to in (None, torch.bfloat16):
            want = P.causal_attention(q, k, v, 0.3, window, round_to)
            for block in (7, 32, 512):
                got = P.causal_attention_blocked(q, k, v, 0.3, window, round_to, block=block)
                assert torch.allclose(got, want, atol=1e-12), (window, round_to, block)
            rows = torch.tensor([3, 74, 20, 21])
            some = P.causal_attention_blocked(q[rows], k, v, 0.3, window, round_to, q_positions=rows, block=3)
            assert torch.allclose(some, want[rows], atol=1e-12)


def test_whole_model_blocked_and_at_chosen_places(tmp_path):
    import tiny_models as TM
    for name in ("A", "C"):
        cfg, w = P.read_model(TM.write_tiny(name, str(tmp_path / name)))
        ids = [int(t) for t in torch.randint(0, cfg["vocab_size"], (45,))]
        full = P.forward(cfg, w, ids)
        assert torch.allclose(P.forward(cfg, w, ids, blocked=True), full, atol=1e-10)
        assert torch.allclose(P.forward(cfg, w, ids, rows=[44, 7, 30]), full[[44, 7, 30]], atol=1e-10)
        assert torch.allclose(P.forward(cfg, w, ids, rows=[0, 5], round_to=torch.bfloat16),
                              P.forward(cfg, w, ids, round_to=torch.bfloat16)[[0, 5]], atol=1e-10)


def test_swiglu_equals_library():
    g, u = torch.randn(4, 10, dtype=torch.float64), torch.randn(4, 10, dtype=torch.float64)
    assert torch.allclose(P.swiglu(g, u), torch.nn.functional.silu(g) * u, atol=1e-12)
    assert not torch.allclose(P.swiglu(g, u), torch.nn.functional.silu(u) * g, atol=1e-3)


def test_linear_layout():
    x, w = torch.randn(3, 5, dtype=torch.float64), torch.randn(7, 5, dtype=torch.float64)
    assert torch.allclose(P.linear(x, w), torch.nn.functional.linear(x, w))


def test_whole_model_position_shift_invariance_of_first_layer_scores(tmp_path):
    """With rotary encoding only distances count: a model run on a sequence gives,
    for its last token, the same logits whether or not a prefix of identical
    tokens is prepended, when attention can only see the last tokens (window)."""
    import tiny_models as TM
    d = TM.write_tiny("C", str(tmp_path / "c"))
    cfg, w = P.read_model(d)
    cfg = dict(cfg, max_window_layers=3)          # every layer windowed
    ids = [int(t) for t in torch.randint(0, cfg["vocab_size"], (70,))]
    # receptive field of 3 windowed layers of window 24: 3 * 23 + 1 = 70 tokens
    a = P.forward(cfg, w, ids)[-1]
    b = P.forward(cfg, w, [7, 9, 11, 13, 5] + ids)[-1]
    assert torch.allclose(a, b, atol=1e-9)


def test_tied_and_untied_heads(tmp_path):
    import tiny_models as TM
    da = TM.write_tiny("A", str(tmp_path / "a"))
    cfg, w = P.read_model(da)
    assert "lm_head.weight" not in w
    ids = [1, 2, 3]
    logits = P.forward(cfg, w, ids)
    w2 = dict(w)
    w2["lm_head.weight"] = w["model.embed_tokens.weight"].clone()
    assert torch.allclose(P.forward(cfg, w2, ids), logits)
    w2["lm_head.weight"] = torch.randn_like(w["model.embed_tokens.weight"])
    assert not torch.allclose(P.forward(cfg, w2, ids), logits)


def test_causality_of_whole_model(tmp_path):
    import tiny_models as TM
    d = TM.write_tiny("B", str(tmp_path / "b"))
    cfg, w = P.read_model(d)
    ids = [int(t) for t in torch.randint(0, cfg["vocab_size"], (20,))]
    full = P.forward(cfg, w, ids)
    part = P.forward(cfg, w, ids[:11])
    assert torch.allclose(full[:11], part, atol=1e-10)


def test_sampler_rules():
    logits = torch.tensor([0.1, 3.0, 2.9, -1.0, 0.5])
    # low temperature: the maximum (sample.rs:176-183)
    for u in (0.0, 0.3, 0.99):
        assert P.sample_token(logits, 1e-4, 0.9, u) == 1
    # nucleus: top_p small keeps only the best token
    assert P.sample_token(logits, 1.0, 0.1, 0.999) == 1
    # top_p = 1: the inverse CDF in the order of the vocabulary
    p = torch.softmax(logits.double(), 0)
    cdf = torch.cumsum(p, 0)
    for u in (0.01, 0.2, 0.5, 0.8, 0.97):
        want = int(torch.nonzero(cdf > u)[0])
        assert P.sample_token(logits, 1.0, 1.0, u) == want
    # penalty: positive logits are divided, negative multiplied (sample.rs:101-112)
    pen = P.sample_token(torch.tensor([2.0, 1.9, -5.0]), 1e-4, 1.0, 0.5, penalty=2.0, recent=[0])
    assert pen == 1
    # same seed, same token index -> same number (sample.rs:167-173)
    assert P.uniform_for_token(42, 3) == P.uniform_for_token(42, 3)
    assert 0.0 <= P.uniform_for_token(42, 0) <= 1.0
    assert P.uniform_for_token(42, 0) != P.uniform_for_token(42, 1)

"""A plain, slow Llama dense decoder: whole sequences, no cache, one function per
part, written from the reference's formulas (each function cites file:line under
the reference's root).  It shares no code with infernum_amd: it reads
config.json with ``json`` and model.safetensors with its own few lines.

Everything is computed in float64 or float32 on the CPU, as asked for by
``dtype``.  Weights are used at the values the file holds (bf16 values are
widened exactly).
"""
from __future__ import annotations

import json
import math
import os
import struct
from typing import Dict, List, Optional, Sequence

import numpy as np
import torch


# ------------------------------------------------------------------------- files
def read_safetensors(path: str) -> Dict[str, torch.Tensor]:
    """name -> CPU tensor.  Format: u64 header length, JSON header, raw bytes."""
    with open(path, "rb") as f:
        (n,) = struct.unpack("<Q", f.read(8))
        header = json.loads(f.read(n))
        data = f.read()
    out = {}
    kinds = {"F32": (np.float32, 4), "F64": (np.float64, 8), "I32": (np.int32, 4), "I64": (np.int64, 8)}
    for name, info in header.items():
        if name == "__metadata__":
            continue
        b, e = info["data_offsets"]
        raw = data[b:e]
        if info["dtype"] == "BF16":
            u16 = np.frombuffer(raw, dtype=np.uint16).astype(np.uint32) << 16
            t = torch.from_numpy(u16.view(np.float32).copy())
        elif info["dtype"] == "F16":
            t = torch.from_numpy(np.frombuffer(raw, dtype=np.float16).astype(np.float32))
        else:
            t = torch.from_numpy(np.frombuffer(raw, dtype=kinds[info["dtype"]][0]).copy())
        out[name] = t.reshape(info["shape"])
    return out


def read_model(model_dir: str):
    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = json.load(f)
    weights = read_safetensors(os.path.join(model_dir, "model.safetensors"))
    return cfg, weights


# ------------------------------------------------------------------------- parts
def embedding(table: torch.Tensor, ids: Sequence[int]) -> torch.Tensor:
    """h[t] = E[ids[t]], no scaling.  infernum-llama/src/graph_builder.rs:442;
    infernum-cuda/kernels/embed.cu:13-16."""
    return table[torch.as_tensor(list(ids), dtype=torch.long)]


def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """x * rsqrt(mean(x^2) + eps) * w: eps inside the root, the weight multiplies.
    infernum-cuda/kernels/rmsnorm.cu:79-80,89-93."""
    ms = (x * x).mean(dim=-1, keepdim=True)
    return x * torch.rsqrt(ms + eps) * w


def linear(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """y = x W^T with W in the file's [out, in] layout, no bias.
    infernum-cuda/src/inner/cuda/ops/linear.rs:10-15; graph_builder.rs:456."""
    return x @ w.t()


def rope_frequencies(head_dim: int, theta: float, scaling: Optional[dict], dtype=torch.float64) -> torch.Tensor:
    """f_i = theta^(-2i/d), i < d/2 (infernum/src/rope.rs:19-30).

    llama3 scaling: the reference's band formula (rope.rs:91-120) with the band
    edges from the configuration: wavelength L = 2 pi / f, original context n;
    L < n/high: f; L > n/low: f/factor; else f(1-r)/factor + f r with
    r = (n/L - low)/(high - low); no magnitude correction.
    """
    i = torch.arange(head_dim // 2, dtype=dtype)
    f = 1.0 / (torch.tensor(theta, dtype=dtype) ** (2.0 * i / head_dim))
    if scaling is None:
        return f
    kind = scaling.get("rope_type", scaling.get("type"))
    assert kind == "llama3", kind
    factor, low, high = scaling["factor"], scaling["low_freq_factor"], scaling["high_freq_factor"]
    n = scaling["original_max_position_embeddings"]
    out = []
    for fi in f.tolist():
        wavelen = 2.0 * math.pi / fi
        if wavelen < n / high:
            out.append(fi)
        elif wavelen > n / low:
            out.append(fi / factor)
        else:
            r = (n / wavelen - low) / (high - low)
            out.append(fi * (1.0 - r) / factor + fi * r)
    return torch.tensor(out, dtype=dtype)


def rope(x: torch.Tensor, positions: torch.Tensor, freqs: torch.Tensor) -> torch.Tensor:
    """x [T, heads, d]; pairs are half-split, (x[i], x[i + d/2]):
    out[i] = x[i] cos a - x[i+d/2] sin a;  out[i+d/2] = x[i] sin a + x[i+d/2] cos a,
    a = position * f_i.  infernum/src/rope.rs:19-30; infernum-cuda/kernels/rope.cu:25-41;
    convention pinned by infernum-cuda/src/inner/cuda/ops/rope.rs:835-885."""
    half = x.shape[-1] // 2
    ang = positions.to(freqs.dtype)[:, None] * freqs[None, :]           # [T, d/2]
    cos, sin = torch.cos(ang).to(x.dtype)[:, None, :], torch.sin(ang).to(x.dtype)[:, None, :]
    a, b = x[..., :half], x[..., half:]
    return torch.cat([a * cos - b * sin, a * sin + b * cos], dim=-1)


def rounded(x: torch.Tensor, to: Optional[torch.dtype]) -> torch.Tensor:
    """x with every value rounded to the nearest of ``to`` (kept in x's own dtype); x itself without ``to``."""
    return x if to is None else x.to(to).to(x.dtype)


def causal_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float,
                     window: Optional[int] = None, round_to: Optional[torch.dtype] = None) -> torch.Tensor:
    """q [T, nh, d], k, v [T, nkv, d] of one whole sequence -> [T, nh, d].

    Query head h reads key/value head h * nkv // nh
    (infernum-cuda/kernels/paged_decode_attention.cu:342); scores scale * <q, k_j>
    over keys j <= t, and j >= t - window + 1 with a window
    (kernels/flash_prefill_attention_v2.cu:85-88); softmax with the maximum
    subtracted; output sum_j w_j v_j.  With ``round_to`` the exponentials are rounded before they
    are summed and multiplied with the values, as a kernel does that feeds them to a matrix unit
    (the reference's kernels keep them in fp32, paged_decode_attention.cu:540-644).
    """
    T, nh, d = q.shape
    nkv = k.shape[1]
    out = torch.zeros_like(q)
    for h in range(nh):
        g = h * nkv // nh
        for t in range(T):
            lo = 0 if not window else max(0, t - window + 1)
            s = (k[lo:t + 1, g, :] @ q[t, h, :]) * scale
            w = rounded(torch.exp(s - s.max()), round_to)
            out[t, h, :] = (w @ v[lo:t + 1, g, :]) / w.sum()
    return out


def causal_attention_blocked(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float,
                             window: Optional[int] = None, round_to: Optional[torch.dtype] = None,
                             q_positions: Optional[torch.Tensor] = None, block: int = 512) -> torch.Tensor:
    """What :func:`causal_attention` computes (the same formulas and citations), one head and a block of query
    rows at a time, so that sequences of thousands of tokens take seconds; ``test_plain_pins`` holds the two
    together.  ``q_positions`` [Tq]: q holds the queries of these places only (default: of every place)."""
    Tq, nh, d = q.shape
    nkv = k.shape[1]
    pos = torch.arange(Tq) if q_positions is None else torch.as_tensor(q_positions, dtype=torch.long)
    out = torch.zeros_like(q)
    for h in range(nh):
        g = h * nkv // nh
        for r0 in range(0, Tq, block):
            p = pos[r0:r0 + block]
            hi = int(p.max()) + 1
            lo = 0 if not window else max(0, int(p.min()) - window + 1)
            s = (q[r0:r0 + block, h, :] @ k[lo:hi, g, :].t()) * scale          # [rows, keys lo .. hi-1]
            j = torch.arange(lo, hi)[None, :]
            seen = j <= p[:, None]
            if window:
                seen &= j >= (p[:, None] - window + 1)
            s = s.masked_fill(~seen, float("-inf"))
            w = rounded(torch.exp(s - s.max(dim=1, keepdim=True).values), round_to)
            out[r0:r0 + block, h, :] = (w @ v[lo:hi, g, :]) / w.sum(dim=1, keepdim=True)
    return out


def swiglu(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """gate / (1 + exp(-gate)) * up.  infernum-cuda/kernels/silu.cu:36-40."""
    return gate / (1.0 + torch.exp(-gate)) * up


# ------------------------------------------------------------------------- model
def layer_window(cfg: dict, layer: int) -> Optional[int]:
    """infernum-llama/src/config.rs:166-179."""
    if not cfg.get("use_sliding_window", False):
        return None
    mwl = cfg.get("max_window_layers")
    if mwl is not None and layer >= mwl:
        return None
    return cfg.get("sliding_window")


def forward(cfg: dict, w: Dict[str, torch.Tensor], ids: Sequence[int], dtype=torch.float64,
            round_to: Optional[torch.dtype] = None, blocked: bool = False,
            rows: Optional[Sequence[int]] = None) -> torch.Tensor:
    """Logits [T, V] of one whole sequence.  Order of operations:
    infernum-llama/src/graph_builder.rs:442-536.

    ``blocked``: attention by :func:`causal_attention_blocked` (long sequences).  ``rows``: logits at these
    places only, [len(rows), V]: the last layer works out its queries, its feed-forward and the head for them
    alone (its keys and values still come from every token), which is what makes a sequence of tens of
    thousands of tokens affordable when only its end is compared.

    ``round_to`` (torch.bfloat16) rounds every activation that an engine serving in that type stores between
    two operations: the outputs of norms, projections, the rotation, attention (and its exponentials), the
    activation function, as the reference's bf16 path does (one rounding at each kernel's store,
    infernum-cuda/kernels/rmsnorm.cu:314, matmul.rs:111); the residual stream and the logits stay unrounded.
    It tells how far rounding alone takes the logits from the exact ones."""
    W = {k: v.to(dtype) for k, v in w.items()}
    r = lambda t: rounded(t, round_to)      # noqa: E731
    nh = cfg["num_attention_heads"]
    nkv = cfg.get("num_key_value_heads") or nh
    H = cfg["hidden_size"]
    d = cfg.get("head_dim") or H // nh
    eps = cfg.get("rms_norm_eps", 1e-5)
    theta = cfg.get("rope_theta", 10000.0)
    freqs = rope_frequencies(d, theta, cfg.get("rope_scaling"), dtype=dtype)
    T = len(ids)
    pos = torch.arange(T)
    keep = None if rows is None else torch.as_tensor(list(rows), dtype=torch.long)
    L = cfg["num_hidden_layers"]
    h = embedding(W["model.embed_tokens.weight"], ids)
    for i in range(L):
        p = f"model.layers.{i}."
        n = r(rms_norm(h, W[p + "input_layernorm.weight"], eps))
        k = r(linear(n, W[p + "self_attn.k_proj.weight"])).reshape(T, nkv, d)
        v = r(linear(n, W[p + "self_attn.v_proj.weight"])).reshape(T, nkv, d)
        k = r(rope(k, pos, freqs))
        q_pos = pos
        if keep is not None and i == L - 1:         # from here on only the wanted places
            n, h, q_pos = n[keep], h[keep], keep
        q = r(linear(n, W[p + "self_attn.q_proj.weight"])).reshape(len(q_pos), nh, d)
        q = r(rope(q, q_pos, freqs))
        if blocked or len(q_pos) != T:
            a = causal_attention_blocked(q, k, v, 1.0 / math.sqrt(d), layer_window(cfg, i), round_to, q_pos)
        else:
            a = causal_attention(q, k, v, 1.0 / math.sqrt(d), layer_window(cfg, i), round_to)
        a = r(a).reshape(len(q_pos), nh * d)
        h = h + r(linear(a, W[p + "self_attn.o_proj.weight"]))
        m = r(rms_norm(h, W[p + "post_attention_layernorm.weight"], eps))
        act = r(swiglu(r(linear(m, W[p + "mlp.gate_proj.weight"])), r(linear(m, W[p + "mlp.up_proj.weight"]))))
        h = h + r(linear(act, W[p + "mlp.down_proj.weight"]))
    f = r(rms_norm(h, W["model.norm.weight"], eps))
    # the head is the embedding matrix when the file has no lm_head.weight
    # (infernum-cuda/src/inner/cuda_graph_engine.rs:225-232)
    head = W["lm_head.weight"] if "lm_head.weight" in W else W["model.embed_tokens.weight"]
    return linear(f, head)


def greedy(cfg: dict, w: Dict[str, torch.Tensor], prompt: Sequence[int], n_new: int,
           eos: Optional[int] = None, dtype=torch.float64) -> List[int]:
    """Greedy continuation by recomputing the whole sequence each time; the lowest
    index wins a tie; the end-of-sequence token stops and is not emitted
    (infernum-runtime/src/engine.rs:453-459)."""
    ids = list(prompt)
    out: List[int] = []
    for _ in range(n_new):
        logits = forward(cfg, w, ids, dtype)[-1]
        tok = int(torch.argmax(logits))     # torch returns the first maximum
        if eos is not None and tok == eos:
            break
        out.append(tok)
        ids.append(tok)
    return out


def greedy_shortfalls(cfg: dict, w: Dict[str, torch.Tensor], prompt: Sequence[int], tokens: Sequence[int],
                      dtype=torch.float64) -> List[float]:
    """For a continuation that somebody else chose greedily: for each of its tokens, how far the plain model's
    logit of that token lies below the plain model's largest logit at that place, as a fraction of the RMS of
    the logits there (0: the plain model's own choice).  An engine whose logits are within e of the plain
    model's can only choose tokens with a shortfall of at most 2 e."""
    ids = list(prompt) + list(tokens)
    logits = forward(cfg, w, ids, dtype)
    out = []
    for i, t in enumerate(tokens):
        row = logits[len(prompt) + i - 1]
        out.append(float((row.max() - row[t]) / row.pow(2).mean().sqrt()))
    return out


# ---------------------------------------------------------------------- sampling
def xorshift64(s: int) -> int:
    """One round of the reference's generator (infernum-runtime/src/engine.rs:491-494)."""
    m = (1 << 64) - 1
    s ^= (s << 13) & m
    s ^= s >> 7
    s ^= (s << 17) & m
    return s


def uniform_for_token(seed: int, generated_before: int) -> float:
    """The uniform number of a request's next token: the per-token state is one
    round over seed ^ generated_before (engine.rs:283,406,491-494); the draw adds
    one, runs four rounds and divides by 2^64 - 1 in f32
    (infernum-cuda/src/inner/cuda/ops/sample.rs:141-147)."""
    m = (1 << 64) - 1
    state = xorshift64((seed ^ generated_before) & m)
    state = (state + 1) & m
    for _ in range(4):
        state = xorshift64(state)
    return float(np.float32(state) / np.float32(m))


def sample_token(logits: torch.Tensor, temperature: float, top_p: float, u: float,
                 penalty: float = 1.0, recent: Sequence[int] = ()) -> int:
    """Penalty, temperature, softmax, nucleus, inverse CDF
    (infernum-cuda/src/inner/cuda/ops/sample.rs:94-159), with two stated
    differences of this engine: the nucleus takes all tokens that tie with the
    one that crosses top_p, and the CDF walks the nucleus in the order of the
    vocabulary instead of by falling probability."""
    x = logits.to(torch.float64).clone()
    if abs(penalty - 1.0) > 1e-7:
        for t in recent:
            x[t] = x[t] / penalty if x[t] > 0 else x[t] * penalty
    x = x / temperature
    e = torch.exp(x - x.max())
    if top_p < 1.0:
        srt, _ = torch.sort(e, descending=True)
        cum = torch.cumsum(srt, 0)
        cross = int(torch.nonzero(cum >= top_p * e.sum())[0])
        keep = e >= srt[cross]
    else:
        keep = torch.ones_like(e, dtype=torch.bool)
    mass = torch.where(keep, e, torch.zeros_like(e))
    cdf = torch.cumsum(mass, 0)
    t = u * cdf[-1]
    idx = torch.nonzero((cdf > t) & keep)
    if len(idx) == 0:
        return int(torch.nonzero(keep)[-1])
    return int(idx[0])

"""A mixer that the framework does not know, with per-request state of its own, defined here,
registered, built into a model beside attention layers, loaded from a model folder and stepped:
without a change to the framework's files.  The schedule names layers twice and lets one run read
another run's cache."""
import math
from dataclasses import dataclass

import pytest
import torch

import plain_llama as P
import trace_tools as TT
from infernum_amd import CacheConfig, Engine, register_architecture, register_part
from infernum_amd.parts import (LayerSpec, Mixer, ModelSpec, PartSpec, ScheduleEntry, StateSpec, WeightSpec)
from infernum_amd.weights import write_random_model

pytestmark = pytest.mark.gpu


class EmaMixer(Mixer):
    """s_t = decay * s_{t-1} + W_in x_t (per request, s_{-1} = 0);  y_t = W_out s_t.
    The state s has a fixed size; it lives in the cache manager's state slots."""

    def __init__(self, rt, hidden_size, state_size):
        super().__init__(rt)
        self.H, self.S = hidden_size, state_size

    def state_spec(self):
        return StateSpec((self.S,))

    def weights(self):
        return {"in_proj.weight": WeightSpec((self.S, self.H), ("normal", 0.2)),
                "out_proj.weight": WeightSpec((self.H, self.S), ("normal", 0.2)),
                "decay": WeightSpec((self.S,), ("uniform", 0.5, 0.95), follows_compute_dtype=False)}

    def load(self, tensors):
        self.w_in, self.w_out, self.decay = tensors["in_proj.weight"], tensors["out_proj.weight"], tensors["decay"]

    def forward(self, x, ctx, cache):
        assert cache.state is not None and cache.k_pages is None
        u = (x.float() @ self.w_in.float().t())
        s_all = torch.empty_like(u)
        slots = ctx.state_slots.tolist()
        row = 0
        for b, n in enumerate(ctx.q_lens):
            s = cache.state[slots[b]]
            for _ in range(n):
                s = self.decay.float() * s + u[row]
                s_all[row] = s
                row += 1
            cache.state[slots[b]] = s
        return (s_all @ self.w_out.float().t()).to(x.dtype)


@dataclass(frozen=True)
class ToyConfig:
    vocab_size: int = 90
    hidden_size: int = 48
    state_size: int = 20
    num_heads: int = 3
    num_kv_heads: int = 1
    intermediate_size: int = 72
    eps: float = 1e-5
    theta: float = 1000.0
    model_type: str = "toy-ema"

    @staticmethod
    def from_dict(raw, where="config.json"):
        return ToyConfig(**{k: v for k, v in raw.items() if k in ToyConfig.__dataclass_fields__})

    def to_dict(self):
        return dict(self.__dict__)


SCHEDULE = [ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(0, cache_of=0), ScheduleEntry(1), ScheduleEntry(2)]


def toy_spec(cfg: ToyConfig) -> ModelSpec:
    H, d = cfg.hidden_size, cfg.hidden_size // cfg.num_heads
    norm = lambda prefix: PartSpec("rmsnorm", {"size": H, "eps": cfg.eps, "init": ("uniform", 0.5, 1.5)}, prefix)
    ff = lambda prefix: PartSpec("swiglu", {"hidden_size": H, "intermediate_size": cfg.intermediate_size,
                                            "init_std": 0.1}, prefix)
    att = lambda prefix, window: PartSpec("attention", {
        "hidden_size": H, "num_heads": cfg.num_heads, "num_kv_heads": cfg.num_kv_heads, "head_dim": d,
        "window": window, "init_std": 0.1,
        "position": {"kind": "rope", "params": {"head_dim": d, "theta": cfg.theta, "scaling": None}}}, prefix)
    ema = lambda prefix: PartSpec("ema", {"hidden_size": H, "state_size": cfg.state_size}, prefix)
    layers = []
    for i, mixer in enumerate([att("layers.0.attn.", None), ema("layers.1.ema."), att("layers.2.attn.", 9)]):
        layers.append(LayerSpec("prenorm", mixer, ff(f"layers.{i}.ff."), norm(f"layers.{i}.norm1."),
                                norm(f"layers.{i}.norm2.")))
    return ModelSpec(vocab_size=cfg.vocab_size, hidden_size=H,
                     embedding=PartSpec("token", {"vocab_size": cfg.vocab_size, "hidden_size": H, "init_std": 0.5},
                                        "embed."),
                     layers=layers, schedule=SCHEDULE, final_norm=norm("final_norm."),
                     head=PartSpec("linear", {"vocab_size": cfg.vocab_size, "hidden_size": H, "init_std": 0.1}, "head."))


def plain_forward(cfg: ToyConfig, w, ids):
    """The toy model on a whole sequence, from the plain functions."""
    W = {k: v.double() for k, v in w.items()}
    H, nh, nkv = cfg.hidden_size, cfg.num_heads, cfg.num_kv_heads
    d = H // nh
    T = len(ids)
    freqs, pos = P.rope_frequencies(d, cfg.theta, None), torch.arange(T)
    h = P.embedding(W["embed.weight"], ids)
    kept = {}
    for e_idx, e in enumerate(SCHEDULE):
        i = e.layer
        n = P.rms_norm(h, W[f"layers.{i}.norm1.weight"], cfg.eps)
        if i == 1:
            p = "layers.1.ema."
            u = P.linear(n, W[p + "in_proj.weight"])
            s, rows = torch.zeros(cfg.state_size, dtype=torch.float64), []
            for t in range(T):
                s = W[p + "decay"] * s + u[t]
                rows.append(s)
            a = P.linear(torch.stack(rows), W[p + "out_proj.weight"])
        else:
            p = f"layers.{i}.attn."
            q = P.rope(P.linear(n, W[p + "q_proj.weight"]).reshape(T, nh, d), pos, freqs)
            if e.cache_of is None:
                k = P.rope(P.linear(n, W[p + "k_proj.weight"]).reshape(T, nkv, d), pos, freqs)
                v = P.linear(n, W[p + "v_proj.weight"]).reshape(T, nkv, d)
                kept[e_idx] = (k, v)
            else:
                k, v = kept[e.cache_of]
            a = P.linear(P.causal_attention(q, k, v, 1.0 / math.sqrt(d), 9 if i == 2 else None).reshape(T, H),
                         W[p + "o_proj.weight"])
        h = h + a
        m = P.rms_norm(h, W[f"layers.{i}.norm2.weight"], cfg.eps)
        h = h + P.linear(P.swiglu(P.linear(m, W[f"layers.{i}.ff.gate_proj.weight"]),
                                  P.linear(m, W[f"layers.{i}.ff.up_proj.weight"])),
                         W[f"layers.{i}.ff.down_proj.weight"])
    return P.linear(P.rms_norm(h, W["final_norm.weight"], cfg.eps), W["head.weight"])


@pytest.fixture(scope="module")
def toy(tmp_path_factory):
    register_part("mixer", "ema", EmaMixer, replace=True)
    register_architecture("toy-ema", ToyConfig, toy_spec, replace=True)
    out = {}
    for dt, tdt in (("float32", torch.float32), ("bfloat16", torch.bfloat16)):
        d = str(tmp_path_factory.mktemp(f"toy_{dt}"))
        write_random_model(ToyConfig(), d, seed=4, dtype=tdt)
        out[dt] = d
    return out


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_model_is_registered_built_loaded_and_stepped(toy, dtype):
    d = toy[dtype]
    cfg = ToyConfig()
    _, w = P.read_model(d)
    assert "layers.1.ema.decay" in w
    eng = Engine.from_pretrained(d, dtype=dtype, cache_config=CacheConfig(page_size=4, num_pages=48,
                                                                          num_state_slots=4, poison_freed_pages=True))
    assert eng.config == cfg
    kinds = [type(b.mixer).__name__ for b in eng.model.blocks]
    assert kinds == ["Attention", "EmaMixer", "Attention"]
    # groups: all keys (layer 0), a window of 9 (layer 2); the ema runs have state and no pages
    assert len(eng.cache.groups) == 2
    assert [v.state is not None for v in eng.views] == [False, True, False, True, False]
    assert eng.views[2].writable is False and eng.views[2].k_pages is eng.views[0].k_pages
    reqs = TT.make_requests(cfg.vocab_size, (37, 5, 60, 23), seed=2)
    ref = {r: plain_forward(cfg, w, t) for r, t in reqs.items()}
    tol = {"float32": 3e-5, "bfloat16": 8e-2}[dtype]
    for name, steps in (("whole", TT.trace_whole(reqs)), ("tail", TT.trace_tail_one_by_one(reqs, 16)),
                        ("portions", TT.trace_portions(reqs)),
                        ("mixed", TT.trace_mixed(reqs, {r: max(2, len(t) - 8) for r, t in reqs.items()}, seed=1)[0])):
        got = TT.run_steps(eng, steps)
        worst, rms, where = TT.error_against(got, ref)
        print(f"toy {dtype} {name}: {worst / rms:.2e} at {where}")
        assert worst == worst and worst <= tol * rms, (name, worst / rms, where)
        eng.cache.check()
        assert eng.cache.slots.num_free == 4 and all(g.allocator.num_free == 48 for g in eng.cache.groups)
    # the step ran as one program: the stock parts' launches made by the host library, the mixer of this file
    # called back in its place among them; the parts' own forward, call by call from Python, gives the same bits
    assert eng.program is not None and eng.program.num_ops > 30 and eng.program.num_python_ops > 0
    twin = Engine.from_pretrained(d, dtype=dtype, executor="parts",
                                  cache_config=CacheConfig(page_size=4, num_pages=48, num_state_slots=4))
    assert twin.program is None
    a, b = TT.run_steps(eng, TT.trace_portions(reqs)), TT.run_steps(twin, TT.trace_portions(reqs))
    assert a.keys() == b.keys() and all(torch.equal(a[k], b[k]) for k in a)


def test_state_slot_is_zeroed_when_taken_again(toy):
    """A request that takes the slot of a finished one must not see its state."""
    eng = Engine.from_pretrained(toy["float32"], dtype="float32",
                                 cache_config=CacheConfig(page_size=4, num_pages=16, num_state_slots=1))
    from infernum_amd import StepEntry
    a = eng.step([StepEntry("a", [1, 2, 3, 4, 5], [4])]).cpu()
    eng.end("a")
    eng.step([StepEntry("b", [9, 8, 7, 6, 5, 4, 3], [])])
    eng.end("b")
    again = eng.step([StepEntry("c", [1, 2, 3, 4, 5], [4])]).cpu()
    assert torch.equal(a, again)


# ------------------------------------------------------------------------------------------------
# A feed-forward with routing and another position encoding, again defined here and not in the framework.
from infernum_amd.parts import FeedForward, PositionEncoding        # noqa: E402


class RoutedFeedForward(FeedForward):
    """Two experts, the one with the larger router logit (fp32) serves the token:
    y = swiglu_e(x), e = argmax(x W_r^T).  Written with torch operations: it is a toy."""

    def __init__(self, rt, hidden_size, intermediate_size, num_experts=2):
        super().__init__(rt)
        self.H, self.I, self.E = hidden_size, intermediate_size, num_experts

    def weights(self):
        w = {"router.weight": WeightSpec((self.E, self.H), ("normal", 0.5), follows_compute_dtype=False)}
        for e in range(self.E):
            w[f"experts.{e}.gate_up.weight"] = WeightSpec((2 * self.I, self.H), ("normal", 0.1))
            w[f"experts.{e}.down.weight"] = WeightSpec((self.H, self.I), ("normal", 0.1))
        return w

    def load(self, tensors):
        self.t = tensors

    def forward(self, x, ctx):
        logits = x.float() @ self.t["router.weight"].float().t()
        choice = logits.argmax(dim=-1)
        out = torch.zeros_like(x)
        for e in range(self.E):
            rows = (choice == e).nonzero().flatten()
            if rows.numel():
                gu = x[rows].float() @ self.t[f"experts.{e}.gate_up.weight"].float().t()
                g, u = gu[:, :self.I], gu[:, self.I:]
                act = (g / (1 + torch.exp(-g)) * u).to(x.dtype)
                out[rows] = (act.float() @ self.t[f"experts.{e}.down.weight"].float().t()).to(x.dtype)
        return out


class SlowedPartialRotary(PositionEncoding):
    """Rotates the first half of each head only, with every frequency divided by ``slow``: what the attention
    kernels need of a position encoding is its table of frequencies and how many values it rotates."""
    graph_safe = True

    def __init__(self, rt, head_dim, theta, slow):
        super().__init__(rt)
        self.rotary_dim = head_dim // 2
        i = torch.arange(self.rotary_dim // 2, dtype=torch.float64)
        self.inv_freq = (theta ** (-2.0 * i / self.rotary_dim) / slow).to(torch.float32).to(rt.device)


@dataclass(frozen=True)
class Toy2Config:
    vocab_size: int = 77
    hidden_size: int = 64
    num_heads: int = 2
    intermediate_size: int = 40
    slow: float = 4.0
    model_type: str = "toy-routed"

    @staticmethod
    def from_dict(raw, where="config.json"):
        return Toy2Config(**{k: v for k, v in raw.items() if k in Toy2Config.__dataclass_fields__})

    def to_dict(self):
        return dict(self.__dict__)


def toy2_spec(cfg: Toy2Config) -> ModelSpec:
    H, d = cfg.hidden_size, cfg.hidden_size // cfg.num_heads
    norm = lambda prefix: PartSpec("rmsnorm", {"size": H, "eps": 1e-5, "init": ("uniform", 0.5, 1.5)}, prefix)
    layers = []
    for i in range(2):
        layers.append(LayerSpec(
            "prenorm",
            PartSpec("attention", {"hidden_size": H, "num_heads": cfg.num_heads, "num_kv_heads": cfg.num_heads,
                                   "head_dim": d, "init_std": 0.1,
                                   "position": {"kind": "slowed_partial_rope",
                                                "params": {"head_dim": d, "theta": 100.0, "slow": cfg.slow}}},
                     f"l.{i}.attn."),
            PartSpec("routed", {"hidden_size": H, "intermediate_size": cfg.intermediate_size}, f"l.{i}.moe.")
            if i == 1 else PartSpec("swiglu", {"hidden_size": H, "intermediate_size": cfg.intermediate_size,
                                               "init_std": 0.1}, f"l.{i}.ff."),
            norm(f"l.{i}.n1."), norm(f"l.{i}.n2.")))
    return ModelSpec(vocab_size=cfg.vocab_size, hidden_size=H,
                     embedding=PartSpec("token", {"vocab_size": cfg.vocab_size, "hidden_size": H, "init_std": 0.5}, "emb."),
                     layers=layers, schedule=[ScheduleEntry(0), ScheduleEntry(1)], final_norm=norm("fn."),
                     head=PartSpec("linear", {"vocab_size": cfg.vocab_size, "hidden_size": H, "init_std": 0.1}, "head."))


def plain_forward2(cfg: Toy2Config, w, ids):
    W = {k: v.double() for k, v in w.items()}
    H, nh = cfg.hidden_size, cfg.num_heads
    d = H // nh
    rot = d // 2
    T = len(ids)
    i = torch.arange(rot // 2, dtype=torch.float64)
    freqs = (100.0 ** (-2.0 * i / rot) / cfg.slow).to(torch.float32).double()
    pos = torch.arange(T)
    h = P.embedding(W["emb.weight"], ids)
    for l in range(2):
        n = P.rms_norm(h, W[f"l.{l}.n1.weight"], 1e-5)
        p = f"l.{l}.attn."
        q = P.linear(n, W[p + "q_proj.weight"]).reshape(T, nh, d)
        k = P.linear(n, W[p + "k_proj.weight"]).reshape(T, nh, d)
        v = P.linear(n, W[p + "v_proj.weight"]).reshape(T, nh, d)
        q = torch.cat([P.rope(q[..., :rot], pos, freqs), q[..., rot:]], -1)
        k = torch.cat([P.rope(k[..., :rot], pos, freqs), k[..., rot:]], -1)
        a = P.causal_attention(q, k, v, 1.0 / math.sqrt(d)).reshape(T, H)
        h = h + P.linear(a, W[p + "o_proj.weight"])
        m = P.rms_norm(h, W[f"l.{l}.n2.weight"], 1e-5)
        if l == 0:
            h = h + P.linear(P.swiglu(P.linear(m, W["l.0.ff.gate_proj.weight"]), P.linear(m, W["l.0.ff.up_proj.weight"])),
                             W["l.0.ff.down_proj.weight"])
        else:
            choice = P.linear(m, W["l.1.moe.router.weight"]).argmax(-1)
            out = torch.zeros_like(m)
            for t in range(T):
                e = int(choice[t])
                gu = P.linear(m[t:t + 1], W[f"l.1.moe.experts.{e}.gate_up.weight"])
                I = cfg.intermediate_size
                out[t] = P.linear(P.swiglu(gu[:, :I], gu[:, I:]), W[f"l.1.moe.experts.{e}.down.weight"])[0]
            h = h + out
    return P.linear(P.rms_norm(h, W["fn.weight"], 1e-5), W["head.weight"])


def test_routed_feed_forward_and_another_position_encoding(tmp_path):
    register_part("feed_forward", "routed", RoutedFeedForward, replace=True)
    register_part("position", "slowed_partial_rope", SlowedPartialRotary, replace=True)
    register_architecture("toy-routed", Toy2Config, toy2_spec, replace=True)
    cfg = Toy2Config()
    d = write_random_model(cfg, str(tmp_path / "toy2"), seed=9, dtype=torch.float32)
    _, w = P.read_model(d)
    eng = Engine.from_pretrained(d, dtype="float32", cache_config=CacheConfig(page_size=4, num_pages=64,
                                                                              num_state_slots=4))
    assert not eng.use_graphs                 # the routed feed-forward is not marked as safe to record
    reqs = TT.make_requests(cfg.vocab_size, (41, 9, 30), seed=6)
    ref = {r: plain_forward2(cfg, w, t) for r, t in reqs.items()}
    for name, steps in (("whole", TT.trace_whole(reqs)), ("portions", TT.trace_portions(reqs)),
                        ("tail", TT.trace_tail_one_by_one(reqs, 10))):
        got = TT.run_steps(eng, steps)
        worst, rms, where = TT.error_against(got, ref)
        print(f"toy2 {name}: {worst / rms:.2e} at {where}")
        assert worst == worst and worst <= 3e-5 * rms, (name, worst / rms, where)


# ------------------------------------------------------------------------------------------------
# A mixer whose pages hold one tensor of its own (a latent per token instead of keys and values), in an
# arrangement of its own (mixer and two feed-forwards side by side on one norm): again without a change to
# the framework's files.
from infernum_amd.parts import Block, CacheSpec, PageTensor        # noqa: E402


class LatentMixer(Mixer):
    """c_t = W_c x_t is what a token leaves in the cache (``rank`` numbers);
    y_t = W_o sum_j softmax_j(<W_q x_t, c_j> / sqrt(rank)) c_j over the tokens j <= t of the request (the last
    ``window`` of them when a window is set)."""

    def __init__(self, rt, hidden_size, rank, window=0):
        super().__init__(rt)
        self.H, self.r, self.window = hidden_size, rank, window

    def cache_spec(self):
        return CacheSpec("window" if self.window else "full", window=self.window,
                         payload=(PageTensor("latent", (self.r,), token_axis=0, dtype=torch.float32),))

    def weights(self):
        return {"c_proj.weight": WeightSpec((self.r, self.H), ("normal", 0.2)),
                "q_proj.weight": WeightSpec((self.r, self.H), ("normal", 0.2)),
                "o_proj.weight": WeightSpec((self.H, self.r), ("normal", 0.2))}

    def load(self, tensors):
        self.t = tensors

    def forward(self, x, ctx, cache):
        pool = cache.pages["latent"]                       # [num_pages, page_size, rank]
        assert cache.k_pages is None and pool.dtype == torch.float32 and pool.shape[2] == self.r
        ps, g = pool.shape[1], cache.group
        flat = pool.view(-1, self.r)
        if cache.writable:                                 # else: the latents of another run of a layer are read
            flat[ctx.slots[g].long()] = x.float() @ self.t["c_proj.weight"].float().t()
        q = x.float() @ self.t["q_proj.weight"].float().t()
        out = torch.empty_like(q)
        tables = ctx.block_tables[g].tolist()
        row = 0
        for b, (n, before) in enumerate(zip(ctx.q_lens, ctx.ctx_lens)):
            for i in range(n):
                t = before + i
                first = max(0, t - self.window + 1) if self.window else 0
                where = torch.tensor([tables[b][p // ps] * ps + p % ps for p in range(first, t + 1)], device=x.device)
                assert int(where.min()) >= 0, "a position inside the window has no page"
                c = flat[where]
                s = torch.softmax(c @ q[row] / math.sqrt(self.r), dim=0)
                out[row] = s @ c
                row += 1
        return (out @ self.t["o_proj.weight"].float().t()).to(x.dtype)


class SideBySideBlock(Block):
    """h += mixer(n) + feed_forward(n) + second(n) with n = norm(h): one norm, nothing in a row."""

    def forward(self, h, pending, ctx, cache):
        n = self.mixer_norm.forward(h, pending)
        parts = [self.mixer.forward(n, ctx, cache), self.feed_forward.forward(n, ctx),
                 self.extra["second"].forward(n, ctx)]
        parts = [p.joined(n.dtype) if hasattr(p, "joined") else p for p in parts]
        return (parts[0].float() + parts[1].float() + parts[2].float()).to(n.dtype)


@dataclass(frozen=True)
class Toy3Config:
    vocab_size: int = 61
    hidden_size: int = 40
    rank: int = 12
    intermediate_size: int = 56
    window: int = 7
    model_type: str = "toy-latent"

    @staticmethod
    def from_dict(raw, where="config.json"):
        return Toy3Config(**{k: v for k, v in raw.items() if k in Toy3Config.__dataclass_fields__})

    def to_dict(self):
        return dict(self.__dict__)


def toy3_spec(cfg: Toy3Config) -> ModelSpec:
    H = cfg.hidden_size
    norm = lambda prefix: PartSpec("rmsnorm", {"size": H, "eps": 1e-5, "init": ("uniform", 0.5, 1.5)}, prefix)
    ff = lambda prefix: PartSpec("swiglu", {"hidden_size": H, "intermediate_size": cfg.intermediate_size,
                                            "init_std": 0.1}, prefix)
    layers = [LayerSpec("side_by_side",
                        PartSpec("latent", {"hidden_size": H, "rank": cfg.rank, "window": w}, f"l.{i}.mix."),
                        ff(f"l.{i}.ff."), norm(f"l.{i}.n."), None,
                        extra={"second": ("feed_forward", ff(f"l.{i}.ff2."))})
              for i, w in enumerate((0, cfg.window))]
    return ModelSpec(vocab_size=cfg.vocab_size, hidden_size=H,
                     embedding=PartSpec("token", {"vocab_size": cfg.vocab_size, "hidden_size": H, "init_std": 0.5}, "emb."),
                     layers=layers, schedule=[ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(0, cache_of=0)],
                     final_norm=norm("fn."),
                     head=PartSpec("linear", {"vocab_size": cfg.vocab_size, "hidden_size": H, "init_std": 0.1}, "head."))


def plain_forward3(cfg: Toy3Config, w, ids):
    W = {k: v.double() for k, v in w.items()}
    T = len(ids)
    h = P.embedding(W["emb.weight"], ids)
    kept = {}
    for run, (l, reads) in enumerate(((0, None), (1, None), (0, 0))):
        n = P.rms_norm(h, W[f"l.{l}.n.weight"], 1e-5)
        if reads is None:
            kept[run] = P.linear(n, W[f"l.{l}.mix.c_proj.weight"])
        c = kept[run if reads is None else reads]
        q = P.linear(n, W[f"l.{l}.mix.q_proj.weight"])
        window = cfg.window if l == 1 else 0
        a = torch.zeros_like(q)
        for t in range(T):
            first = max(0, t - window + 1) if window else 0
            s = torch.softmax(c[first:t + 1] @ q[t] / math.sqrt(cfg.rank), dim=0)
            a[t] = s @ c[first:t + 1]
        delta = P.linear(a, W[f"l.{l}.mix.o_proj.weight"])
        for f in ("ff", "ff2"):
            delta = delta + P.linear(P.swiglu(P.linear(n, W[f"l.{l}.{f}.gate_proj.weight"]),
                                              P.linear(n, W[f"l.{l}.{f}.up_proj.weight"])),
                                     W[f"l.{l}.{f}.down_proj.weight"])
        h = h + delta
    return P.linear(P.rms_norm(h, W["fn.weight"], 1e-5), W["head.weight"])


def test_a_mixer_with_a_page_payload_of_its_own_in_an_arrangement_of_its_own(tmp_path):
    register_part("mixer", "latent", LatentMixer, replace=True)
    register_part("block", "side_by_side", SideBySideBlock, replace=True)
    register_architecture("toy-latent", Toy3Config, toy3_spec, replace=True)
    cfg = Toy3Config()
    d = write_random_model(cfg, str(tmp_path / "toy3"), seed=12, dtype=torch.float32)
    _, w = P.read_model(d)
    eng = Engine.from_pretrained(d, dtype="float32", cache_config=CacheConfig(page_size=4, num_pages=40,
                                                                              num_state_slots=4, poison_freed_pages=True))
    # two groups (all positions; a window of 7), pools as the mixer declared them, the third run reads the first's
    assert [(g.kind, g.window) for g in eng.cache.groups] == [("full", 0), ("window", cfg.window)]
    assert [sorted(p) for p in eng.cache.pages] == [["latent"], ["latent"], []]
    assert tuple(eng.cache.pages[0]["latent"].shape) == (40, 4, cfg.rank)
    assert eng.views[2].pages is eng.views[0].pages and not eng.views[2].writable
    assert eng.model.step_needs() == {} and not eng.use_graphs
    reqs = TT.make_requests(cfg.vocab_size, (33, 6, 50, 21), seed=3)
    ref = {r: plain_forward3(cfg, w, t) for r, t in reqs.items()}
    for name, steps in (("whole", TT.trace_whole(reqs)), ("tail", TT.trace_tail_one_by_one(reqs, 12)),
                        ("portions", TT.trace_portions(reqs)),
                        ("mixed", TT.trace_mixed(reqs, {r: max(2, len(t) - 8) for r, t in reqs.items()}, seed=2)[0])):
        got = TT.run_steps(eng, steps)
        worst, rms, where = TT.error_against(got, ref)
        print(f"toy3 {name}: {worst / rms:.2e} at {where}")
        assert worst == worst and worst <= 3e-5 * rms, (name, worst / rms, where)
        eng.cache.check()
        assert all(g.allocator.num_free == 40 for g in eng.cache.groups)


# ------------------------------------------------------------------------------------------------
# The seam between projection and rotation: a part of the test's own that normalises every query and key head
# (with a weight per position of the head) before they are rotated and the keys are cached.
from infernum_amd.parts import QKTransform        # noqa: E402


class HeadNorm(QKTransform):
    """q_h <- rmsnorm(q_h) * wq, k_h <- rmsnorm(k_h) * wk for every head h; values stay."""

    def __init__(self, rt, head_dim, eps):
        super().__init__(rt)
        self.d, self.eps = head_dim, eps

    def weights(self):
        return {"q_norm.weight": WeightSpec((self.d,), ("uniform", 0.5, 1.5), follows_compute_dtype=False),
                "k_norm.weight": WeightSpec((self.d,), ("uniform", 0.5, 1.5), follows_compute_dtype=False)}

    def load(self, tensors):
        self.wq, self.wk = tensors["q_norm.weight"].float(), tensors["k_norm.weight"].float()

    def forward(self, qkv, num_q_heads, num_kv_heads, head_dim, ctx):
        N = qkv.shape[0]
        heads = qkv.float().view(N, -1, head_dim)
        normed = heads * torch.rsqrt((heads * heads).mean(-1, keepdim=True) + self.eps)
        out = heads.clone()
        out[:, :num_q_heads] = normed[:, :num_q_heads] * self.wq
        out[:, num_q_heads:num_q_heads + num_kv_heads] = normed[:, num_q_heads:num_q_heads + num_kv_heads] * self.wk
        return out.view(N, -1).to(qkv.dtype)


@dataclass(frozen=True)
class Toy4Config:
    vocab_size: int = 70
    hidden_size: int = 64
    num_heads: int = 4
    num_kv_heads: int = 2
    intermediate_size: int = 48
    model_type: str = "toy-headnorm"

    @staticmethod
    def from_dict(raw, where="config.json"):
        return Toy4Config(**{k: v for k, v in raw.items() if k in Toy4Config.__dataclass_fields__})

    def to_dict(self):
        return dict(self.__dict__)


def toy4_spec(cfg: Toy4Config) -> ModelSpec:
    H, d = cfg.hidden_size, cfg.hidden_size // cfg.num_heads
    norm = lambda prefix: PartSpec("rmsnorm", {"size": H, "eps": 1e-5, "init": ("uniform", 0.5, 1.5)}, prefix)
    att = lambda prefix: PartSpec("attention", {
        "hidden_size": H, "num_heads": cfg.num_heads, "num_kv_heads": cfg.num_kv_heads, "head_dim": d, "init_std": 0.2,
        "position": {"kind": "rope", "params": {"head_dim": d, "theta": 1000.0, "scaling": None}},
        "qk_transform": {"kind": "head_norm", "params": {"head_dim": d, "eps": 1e-6}}}, prefix)
    layers = [LayerSpec("prenorm", att(f"l.{i}.attn."),
                        PartSpec("swiglu", {"hidden_size": H, "intermediate_size": cfg.intermediate_size,
                                            "init_std": 0.1}, f"l.{i}.ff."), norm(f"l.{i}.n1."), norm(f"l.{i}.n2."))
              for i in range(2)]
    return ModelSpec(vocab_size=cfg.vocab_size, hidden_size=H,
                     embedding=PartSpec("token", {"vocab_size": cfg.vocab_size, "hidden_size": H, "init_std": 0.5}, "emb."),
                     layers=layers, schedule=[ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(1, cache_of=1)],
                     final_norm=norm("fn."),
                     head=PartSpec("linear", {"vocab_size": cfg.vocab_size, "hidden_size": H, "init_std": 0.1}, "head."))


def plain_forward4(cfg: Toy4Config, w, ids):
    W = {k: v.double() for k, v in w.items()}
    H, nh, nkv = cfg.hidden_size, cfg.num_heads, cfg.num_kv_heads
    d, T = H // nh, len(ids)
    freqs, pos = P.rope_frequencies(d, 1000.0, None), torch.arange(T)
    h = P.embedding(W["emb.weight"], ids)
    kept = {}
    for run, (l, reads) in enumerate(((0, None), (1, None), (1, 1))):
        p = f"l.{l}.attn."
        n = P.rms_norm(h, W[f"l.{l}.n1.weight"], 1e-5)
        q = P.rms_norm(P.linear(n, W[p + "q_proj.weight"]).reshape(T, nh, d), W[p + "q_norm.weight"], 1e-6)
        if reads is None:
            k = P.rms_norm(P.linear(n, W[p + "k_proj.weight"]).reshape(T, nkv, d), W[p + "k_norm.weight"], 1e-6)
            kept[run] = (P.rope(k, pos, freqs), P.linear(n, W[p + "v_proj.weight"]).reshape(T, nkv, d))
        k, v = kept[run if reads is None else reads]
        a = P.causal_attention(P.rope(q, pos, freqs), k, v, 1.0 / math.sqrt(d)).reshape(T, H)
        h = h + P.linear(a, W[p + "o_proj.weight"])
        m = P.rms_norm(h, W[f"l.{l}.n2.weight"], 1e-5)
        h = h + P.linear(P.swiglu(P.linear(m, W[f"l.{l}.ff.gate_proj.weight"]), P.linear(m, W[f"l.{l}.ff.up_proj.weight"])),
                         W[f"l.{l}.ff.down_proj.weight"])
    return P.linear(P.rms_norm(h, W["fn.weight"], 1e-5), W["head.weight"])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_part_between_projection_and_rotation(tmp_path, dtype):
    register_part("qk_transform", "head_norm", HeadNorm, replace=True)
    register_architecture("toy-headnorm", Toy4Config, toy4_spec, replace=True)
    cfg = Toy4Config()
    d = write_random_model(cfg, str(tmp_path / "toy4"), seed=21,
                           dtype={"float32": torch.float32, "bfloat16": torch.bfloat16}[dtype])
    _, w = P.read_model(d)
    assert "l.0.attn.q_norm.weight" in w and "l.1.attn.k_norm.weight" in w      # the transform's tensors, by name
    eng = Engine.from_pretrained(d, dtype=dtype, cache_config=CacheConfig(page_size=8, num_pages=40, num_state_slots=4,
                                                                          poison_freed_pages=True))
    assert eng.program is not None and not eng.use_graphs       # the model's own part is called back from the program; unrecorded
    reqs = TT.make_requests(cfg.vocab_size, (29, 7, 44, 18), seed=5)
    ref = {r: plain_forward4(cfg, w, t) for r, t in reqs.items()}
    tol = {"float32": 3e-5, "bfloat16": 8e-2}[dtype]
    for name, steps in (("whole", TT.trace_whole(reqs)), ("tail", TT.trace_tail_one_by_one(reqs, 12)),
                        ("portions", TT.trace_portions(reqs)),
                        ("mixed", TT.trace_mixed(reqs, {r: max(2, len(t) - 8) for r, t in reqs.items()}, seed=4)[0])):
        got = TT.run_steps(eng, steps)
        worst, rms, where = TT.error_against(got, ref)
        print(f"toy4 {dtype} {name}: {worst / rms:.2e} at {where}")
        assert worst == worst and worst <= tol * rms, (name, worst / rms, where)


# ------------------------------------------------------------------------------------------------
# The remaining kinds of parts as a model's own: a norm (centred, with a bias), an embedding (scaled, with a
# learned vector per position added) and a head (with a cap on the logits) around the stock attention and
# feed-forward.
from infernum_amd.parts import Embedding, Head, Norm        # noqa: E402


class CentredNorm(Norm):
    """out = (s - mean(s)) / sqrt(var(s) + eps) * w + b with s = h + delta."""

    def __init__(self, rt, size, eps):
        super().__init__(rt)
        self.size, self.eps = size, eps

    def weights(self):
        return {"weight": WeightSpec((self.size,), ("uniform", 0.5, 1.5), follows_compute_dtype=False),
                "bias": WeightSpec((self.size,), ("normal", 0.1), follows_compute_dtype=False)}

    def load(self, tensors):
        self.w, self.b = tensors["weight"].float(), tensors["bias"].float()

    def forward(self, h, delta, out=None, rows=None):
        if delta is not None:
            delta = delta.joined(torch.float32) if hasattr(delta, "joined") else delta.float()
        if rows is not None:                               # only these rows, and h stays as it is
            s = h.index_select(0, rows.long())
            if delta is not None:
                s = s + delta.index_select(0, rows.long())
        else:
            if delta is not None:
                h += delta
            s = h
        c = s - s.mean(-1, keepdim=True)
        y = (c * torch.rsqrt(c.pow(2).mean(-1, keepdim=True) + self.eps) * self.w + self.b).to(self.rt.dtype)
        if out is not None:
            out.copy_(y)
            return out
        return y


class ScaledPositionedEmbedding(Embedding):
    """h[t] = sqrt(H) * E[id_t] + P[position_t]."""

    def __init__(self, rt, vocab_size, hidden_size, max_positions):
        super().__init__(rt)
        self.V, self.H, self.L = vocab_size, hidden_size, max_positions

    def weights(self):
        return {"weight": WeightSpec((self.V, self.H), ("normal", 0.3)),
                "positions": WeightSpec((self.L, self.H), ("normal", 0.2))}

    def load(self, tensors):
        self.table, self.pos = tensors["weight"], tensors["positions"]

    def forward(self, ctx):
        return (math.sqrt(self.H) * self.table[ctx.token_ids.long()].float()
                + self.pos[ctx.positions.long()].float()).contiguous()


class CappedHead(Head):
    """logits = cap * tanh(W f / cap)."""

    def __init__(self, rt, vocab_size, hidden_size, cap):
        super().__init__(rt)
        self.V, self.H, self.cap = vocab_size, hidden_size, cap

    def weights(self):
        return {"weight": WeightSpec((self.V, self.H), ("normal", 0.3))}

    def load(self, tensors):
        self.w = tensors["weight"]

    def forward(self, x):
        return self.cap * torch.tanh(x.float() @ self.w.float().t() / self.cap)


@dataclass(frozen=True)
class Toy5Config:
    vocab_size: int = 53
    hidden_size: int = 48
    num_heads: int = 3
    num_kv_heads: int = 1
    intermediate_size: int = 72
    max_positions: int = 96
    cap: float = 5.0
    eps: float = 1e-4
    model_type: str = "toy-dressed"

    @staticmethod
    def from_dict(raw, where="config.json"):
        return Toy5Config(**{k: v for k, v in raw.items() if k in Toy5Config.__dataclass_fields__})

    def to_dict(self):
        return dict(self.__dict__)


def toy5_spec(cfg: Toy5Config) -> ModelSpec:
    H, d = cfg.hidden_size, cfg.hidden_size // cfg.num_heads
    norm = lambda prefix: PartSpec("centred", {"size": H, "eps": cfg.eps}, prefix)
    layers = [LayerSpec("prenorm",
                        PartSpec("attention", {"hidden_size": H, "num_heads": cfg.num_heads, "num_kv_heads": cfg.num_kv_heads,
                                               "head_dim": d, "init_std": 0.1,
                                               "position": {"kind": "none", "params": {}}}, f"l.{i}.attn."),
                        PartSpec("swiglu", {"hidden_size": H, "intermediate_size": cfg.intermediate_size, "init_std": 0.1},
                                 f"l.{i}.ff."),
                        norm(f"l.{i}.n1."), norm(f"l.{i}.n2.")) for i in range(2)]
    return ModelSpec(vocab_size=cfg.vocab_size, hidden_size=H,
                     embedding=PartSpec("scaled_positioned", {"vocab_size": cfg.vocab_size, "hidden_size": H,
                                                              "max_positions": cfg.max_positions}, "emb."),
                     layers=layers, schedule=[ScheduleEntry(0), ScheduleEntry(1)], final_norm=norm("fn."),
                     head=PartSpec("capped", {"vocab_size": cfg.vocab_size, "hidden_size": H, "cap": cfg.cap}, "head."))


def plain_forward5(cfg: Toy5Config, w, ids):
    W = {k: v.double() for k, v in w.items()}
    H, nh, nkv = cfg.hidden_size, cfg.num_heads, cfg.num_kv_heads
    d, T = H // nh, len(ids)

    def centred(x, p):
        c = x - x.mean(-1, keepdim=True)
        return c / torch.sqrt(c.pow(2).mean(-1, keepdim=True) + cfg.eps) * W[p + "weight"] + W[p + "bias"]

    h = math.sqrt(H) * P.embedding(W["emb.weight"], ids) + W["emb.positions"][:T]
    for l in range(2):
        p = f"l.{l}.attn."
        n = centred(h, f"l.{l}.n1.")
        q = P.linear(n, W[p + "q_proj.weight"]).reshape(T, nh, d)
        k = P.linear(n, W[p + "k_proj.weight"]).reshape(T, nkv, d)
        v = P.linear(n, W[p + "v_proj.weight"]).reshape(T, nkv, d)
        h = h + P.linear(P.causal_attention(q, k, v, 1.0 / math.sqrt(d)).reshape(T, H), W[p + "o_proj.weight"])
        m = centred(h, f"l.{l}.n2.")
        h = h + P.linear(P.swiglu(P.linear(m, W[f"l.{l}.ff.gate_proj.weight"]), P.linear(m, W[f"l.{l}.ff.up_proj.weight"])),
                         W[f"l.{l}.ff.down_proj.weight"])
    return cfg.cap * torch.tanh(P.linear(centred(h, "fn."), W["head.weight"]) / cfg.cap)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_norm_an_embedding_and_a_head_of_the_models_own(tmp_path, dtype):
    register_part("norm", "centred", CentredNorm, replace=True)
    register_part("embedding", "scaled_positioned", ScaledPositionedEmbedding, replace=True)
    register_part("head", "capped", CappedHead, replace=True)
    register_architecture("toy-dressed", Toy5Config, toy5_spec, replace=True)
    cfg = Toy5Config()
    d = write_random_model(cfg, str(tmp_path / "toy5"), seed=33,
                           dtype={"float32": torch.float32, "bfloat16": torch.bfloat16}[dtype])
    _, w = P.read_model(d)
    assert {"emb.positions", "fn.bias", "l.1.n2.bias", "head.weight"} <= set(w)
    eng = Engine.from_pretrained(d, dtype=dtype, cache_config=CacheConfig(page_size=4, num_pages=48, num_state_slots=4,
                                                                          poison_freed_pages=True))
    assert eng.program is not None and not eng.use_graphs       # the model's own parts are called back from the program; unrecorded
    reqs = TT.make_requests(cfg.vocab_size, (37, 5, 52, 20), seed=8)
    ref = {r: plain_forward5(cfg, w, t) for r, t in reqs.items()}
    assert max(float(v.abs().max()) for v in ref.values()) <= cfg.cap
    tol = {"float32": 3e-5, "bfloat16": 8e-2}[dtype]
    for name, steps in (("whole", TT.trace_whole(reqs)), ("tail", TT.trace_tail_one_by_one(reqs, 12)),
                        ("portions", TT.trace_portions(reqs)),
                        ("mixed", TT.trace_mixed(reqs, {r: max(2, len(t) - 8) for r, t in reqs.items()}, seed=2)[0])):
        got = TT.run_steps(eng, steps)
        worst, rms, where = TT.error_against(got, ref)
        print(f"toy5 {dtype} {name}: {worst / rms:.2e} at {where}")
        assert worst == worst and worst <= tol * rms, (name, worst / rms, where)


# ------------------------------------------------------------------------------------------------
# Two cached parts in one layer: an attention (pages) and the mixer with state of this file's top side by side,
# each with memory of its own from the cache manager.
class HybridBlock(Block):
    """h += attention(n) + ema(n) with n = norm1(h); then h += feed_forward(norm2(h))."""

    def cached_parts(self):
        return {"mixer": self.mixer, "second": self.extra["second"]}

    def forward(self, h, pending, ctx, cache):
        n = self.mixer_norm.forward(h, pending)
        a = self.mixer.forward(n, ctx, cache)
        a = a.joined(n.dtype) if hasattr(a, "joined") else a
        b = self.extra["second"].forward(n, ctx, cache.others["second"])
        n2 = self.feed_forward_norm.forward(h, (a.float() + b.float()).to(n.dtype))
        return self.feed_forward.forward(n2, ctx)


@dataclass(frozen=True)
class Toy6Config:
    vocab_size: int = 70
    hidden_size: int = 48
    state_size: int = 10
    num_heads: int = 3
    intermediate_size: int = 64
    model_type: str = "toy-hybrid"

    @staticmethod
    def from_dict(raw, where="config.json"):
        return Toy6Config(**{k: v for k, v in raw.items() if k in Toy6Config.__dataclass_fields__})

    def to_dict(self):
        return dict(self.__dict__)


def toy6_spec(cfg: Toy6Config) -> ModelSpec:
    H, d = cfg.hidden_size, cfg.hidden_size // cfg.num_heads
    norm = lambda prefix: PartSpec("rmsnorm", {"size": H, "eps": 1e-5, "init": ("uniform", 0.5, 1.5)}, prefix)
    layers = [LayerSpec("hybrid",
                        PartSpec("attention", {"hidden_size": H, "num_heads": cfg.num_heads, "num_kv_heads": 1,
                                               "head_dim": d, "init_std": 0.1, "position": {
                                                   "kind": "rope", "params": {"head_dim": d, "theta": 1000.0, "scaling": None}}},
                                 f"l.{i}.attn."),
                        PartSpec("swiglu", {"hidden_size": H, "intermediate_size": cfg.intermediate_size, "init_std": 0.1},
                                 f"l.{i}.ff."),
                        norm(f"l.{i}.n1."), norm(f"l.{i}.n2."),
                        extra={"second": ("mixer", PartSpec("ema", {"hidden_size": H, "state_size": cfg.state_size},
                                                            f"l.{i}.ema."))})
              for i in range(2)]
    return ModelSpec(vocab_size=cfg.vocab_size, hidden_size=H,
                     embedding=PartSpec("token", {"vocab_size": cfg.vocab_size, "hidden_size": H, "init_std": 0.5}, "emb."),
                     layers=layers, schedule=[ScheduleEntry(0), ScheduleEntry(1)], final_norm=norm("fn."),
                     head=PartSpec("linear", {"vocab_size": cfg.vocab_size, "hidden_size": H, "init_std": 0.1}, "head."))


def plain_forward6(cfg: Toy6Config, w, ids):
    W = {k: v.double() for k, v in w.items()}
    H, nh = cfg.hidden_size, cfg.num_heads
    d, T = H // nh, len(ids)
    freqs, pos = P.rope_frequencies(d, 1000.0, None), torch.arange(T)
    h = P.embedding(W["emb.weight"], ids)
    for l in range(2):
        n = P.rms_norm(h, W[f"l.{l}.n1.weight"], 1e-5)
        p = f"l.{l}.attn."
        q = P.rope(P.linear(n, W[p + "q_proj.weight"]).reshape(T, nh, d), pos, freqs)
        k = P.rope(P.linear(n, W[p + "k_proj.weight"]).reshape(T, 1, d), pos, freqs)
        v = P.linear(n, W[p + "v_proj.weight"]).reshape(T, 1, d)
        a = P.linear(P.causal_attention(q, k, v, 1.0 / math.sqrt(d)).reshape(T, H), W[p + "o_proj.weight"])
        p = f"l.{l}.ema."
        u = P.linear(n, W[p + "in_proj.weight"])
        s, rows = torch.zeros(cfg.state_size, dtype=torch.float64), []
        for t in range(T):
            s = W[p + "decay"] * s + u[t]
            rows.append(s)
        h = h + a + P.linear(torch.stack(rows), W[p + "out_proj.weight"])
        m = P.rms_norm(h, W[f"l.{l}.n2.weight"], 1e-5)
        h = h + P.linear(P.swiglu(P.linear(m, W[f"l.{l}.ff.gate_proj.weight"]), P.linear(m, W[f"l.{l}.ff.up_proj.weight"])),
                         W[f"l.{l}.ff.down_proj.weight"])
    return P.linear(P.rms_norm(h, W["fn.weight"], 1e-5), W["head.weight"])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_two_cached_parts_side_by_side_in_one_layer(tmp_path, dtype):
    register_part("mixer", "ema", EmaMixer, replace=True)
    register_part("block", "hybrid", HybridBlock, replace=True)
    register_architecture("toy-hybrid", Toy6Config, toy6_spec, replace=True)
    cfg = Toy6Config()
    d = write_random_model(cfg, str(tmp_path / "toy6"), seed=44,
                           dtype={"float32": torch.float32, "bfloat16": torch.bfloat16}[dtype])
    _, w = P.read_model(d)
    eng = Engine.from_pretrained(d, dtype=dtype, cache_config=CacheConfig(page_size=4, num_pages=48, num_state_slots=4,
                                                                          poison_freed_pages=True))
    # per layer the attention's pages and the other mixer's state, each its own
    assert [sorted(p) for p in eng.cache.pages] == [["k", "v"], [], ["k", "v"], []]
    assert [s is not None for s in eng.cache.state] == [False, True, False, True]
    assert all(v.k_pages is not None and v.others["second"].state is not None for v in eng.views)
    assert eng.views[0].others["second"].state is not eng.views[1].others["second"].state
    reqs = TT.make_requests(cfg.vocab_size, (31, 6, 47, 19), seed=6)
    ref = {r: plain_forward6(cfg, w, t) for r, t in reqs.items()}
    tol = {"float32": 3e-5, "bfloat16": 8e-2}[dtype]
    for name, steps in (("whole", TT.trace_whole(reqs)), ("tail", TT.trace_tail_one_by_one(reqs, 12)),
                        ("portions", TT.trace_portions(reqs)),
                        ("mixed", TT.trace_mixed(reqs, {r: max(2, len(t) - 8) for r, t in reqs.items()}, seed=3)[0])):
        got = TT.run_steps(eng, steps)
        worst, rms, where = TT.error_against(got, ref)
        print(f"toy6 {dtype} {name}: {worst / rms:.2e} at {where}")
        assert worst == worst and worst <= tol * rms, (name, worst / rms, where)
        eng.cache.check()
        assert eng.cache.slots.num_free == 4 and all(g.allocator.num_free == 48 for g in eng.cache.groups)


# ------------------------------------------------------------------------------------------------
# A position encoding that rotates neighbouring pairs (x[2i], x[2i + 1]) where the kernels pair the halves of a
# head: it asks the attention for its heads' values in the order [0, 2, 4, ..., 1, 3, 5, ...] and is then served
# by the stock kernels.
class NeighbourPairsRope(PositionEncoding):
    graph_safe = True

    def __init__(self, rt, head_dim, theta):
        super().__init__(rt)
        self.rotary_dim = head_dim
        self.inv_freq = (float(theta) ** (-torch.arange(0, head_dim, 2, dtype=torch.float64) / head_dim)).to(rt.device)

    def head_permutation(self):
        return torch.cat([torch.arange(0, self.rotary_dim, 2), torch.arange(1, self.rotary_dim, 2)])


def _rope_neighbours(x, positions, freqs):
    """x [T, heads, d]: out[2i] = x[2i] cos a - x[2i+1] sin a; out[2i+1] = x[2i] sin a + x[2i+1] cos a, a = p f_i."""
    ang = positions.to(freqs.dtype)[:, None] * freqs[None, :]
    cos, sin = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    a, b = x[..., 0::2], x[..., 1::2]
    out = torch.empty_like(x)
    out[..., 0::2] = a * cos - b * sin
    out[..., 1::2] = a * sin + b * cos
    return out


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_position_encoding_that_pairs_neighbours(tmp_path, dtype):
    register_part("position", "neighbour_pairs", NeighbourPairsRope, replace=True)
    H, nh, nkv, d, V, I = 64, 4, 2, 16, 80, 96

    @dataclass(frozen=True)
    class Toy7Config:
        model_type: str = "toy-neighbours"

        @staticmethod
        def from_dict(raw, where="config.json"):
            return Toy7Config()

        def to_dict(self):
            return {"model_type": self.model_type}

    def spec(cfg):
        norm = lambda prefix: PartSpec("rmsnorm", {"size": H, "eps": 1e-5, "init": ("uniform", 0.5, 1.5)}, prefix)
        layers = [LayerSpec("prenorm",
                            PartSpec("attention", {"hidden_size": H, "num_heads": nh, "num_kv_heads": nkv, "head_dim": d,
                                                   "init_std": 0.15, "position": {"kind": "neighbour_pairs", "params": {
                                                       "head_dim": d, "theta": 100.0}}}, f"l.{i}.attn."),
                            PartSpec("swiglu", {"hidden_size": H, "intermediate_size": I, "init_std": 0.1}, f"l.{i}.ff."),
                            norm(f"l.{i}.n1."), norm(f"l.{i}.n2.")) for i in range(2)]
        return ModelSpec(vocab_size=V, hidden_size=H,
                         embedding=PartSpec("token", {"vocab_size": V, "hidden_size": H, "init_std": 0.5}, "emb."),
                         layers=layers, schedule=[ScheduleEntry(0), ScheduleEntry(1)], final_norm=norm("fn."),
                         head=PartSpec("linear", {"vocab_size": V, "hidden_size": H, "init_std": 0.1}, "head."))

    register_architecture("toy-neighbours", Toy7Config, spec, replace=True)
    folder = write_random_model(Toy7Config(), str(tmp_path / "toy7"), seed=51,
                                dtype={"float32": torch.float32, "bfloat16": torch.bfloat16}[dtype])
    _, w = P.read_model(folder)

    def plain(ids):
        W = {k: v.double() for k, v in w.items()}
        T = len(ids)
        freqs, pos = 100.0 ** (-torch.arange(0, d, 2, dtype=torch.float64) / d), torch.arange(T)
        h = P.embedding(W["emb.weight"], ids)
        for l in range(2):
            n = P.rms_norm(h, W[f"l.{l}.n1.weight"], 1e-5)
            p = f"l.{l}.attn."
            q = _rope_neighbours(P.linear(n, W[p + "q_proj.weight"]).reshape(T, nh, d), pos, freqs)
            k = _rope_neighbours(P.linear(n, W[p + "k_proj.weight"]).reshape(T, nkv, d), pos, freqs)
            v = P.linear(n, W[p + "v_proj.weight"]).reshape(T, nkv, d)
            h = h + P.linear(P.causal_attention(q, k, v, 1.0 / math.sqrt(d)).reshape(T, nh * d), W[p + "o_proj.weight"])
            m = P.rms_norm(h, W[f"l.{l}.n2.weight"], 1e-5)
            h = h + P.linear(P.swiglu(P.linear(m, W[f"l.{l}.ff.gate_proj.weight"]), P.linear(m, W[f"l.{l}.ff.up_proj.weight"])),
                             W[f"l.{l}.ff.down_proj.weight"])
        return P.linear(P.rms_norm(h, W["fn.weight"], 1e-5), W["head.weight"])

    # the pairing matters: the stock half-split rotation of the same weights gives other logits
    ids = [3, 9, 27, 1, 60, 44, 12]
    halves = P.rope(torch.ones(7, 1, d, dtype=torch.float64), torch.arange(7), 100.0 ** (-torch.arange(0, d, 2, dtype=torch.float64) / d))
    assert not torch.allclose(halves, _rope_neighbours(torch.ones(7, 1, d, dtype=torch.float64), torch.arange(7),
                                                       100.0 ** (-torch.arange(0, d, 2, dtype=torch.float64) / d)))
    eng = Engine.from_pretrained(folder, dtype=dtype, cache_config=CacheConfig(page_size=4, num_pages=48, num_state_slots=4,
                                                                               poison_freed_pages=True))
    assert eng.use_graphs                                  # nothing of the model's own runs on the host
    reqs = TT.make_requests(V, (33, 6, 41, 20), seed=9)
    ref = {r: plain(t) for r, t in reqs.items()}
    tol = {"float32": 3e-5, "bfloat16": 8e-2}[dtype]
    for name, steps in (("whole", TT.trace_whole(reqs)), ("tail", TT.trace_tail_one_by_one(reqs, 12)),
                        ("portions", TT.trace_portions(reqs)),
                        ("mixed", TT.trace_mixed(reqs, {r: max(2, len(t) - 8) for r, t in reqs.items()}, seed=5)[0])):
        got = TT.run_steps(eng, steps)
        worst, rms, where = TT.error_against(got, ref)
        print(f"toy7 {dtype} {name}: {worst / rms:.2e} at {where}")
        assert worst == worst and worst <= tol * rms, (name, worst / rms, where)


# ------------------------------------------------------------------------------------------------
# A feed-forward of the test's own that writes its own launches into the step's program (two products through a
# narrow middle, y = W_out (W_in x), no activation), so that no operation of the program calls back into Python:
# the part uses the framework's products and intermediates, and nothing under the framework's folders changes.
class BottleneckFeedForward(FeedForward):
    graph_safe = True

    def __init__(self, rt, hidden_size, rank):
        super().__init__(rt)
        self.H, self.r = hidden_size, rank

    def weights(self):
        return {"in.weight": WeightSpec((self.r, self.H), ("normal", 0.2)),
                "out.weight": WeightSpec((self.H, self.r), ("normal", 0.2))}

    def load(self, tensors):
        self.w_in, self.w_out = tensors["in.weight"].contiguous(), tensors["out.weight"].contiguous()

    def forward(self, x, ctx=None):
        from infernum_amd.parts.linear import linear
        return linear(linear(x, self.w_in, kernels=self.rt.kernels), self.w_out, keep_split=True, kernels=self.rt.kernels)

    def native(self, program, view=None):
        from infernum_amd.parts.linear import emit_linear
        dt = self.rt.dtype
        mid = emit_linear(program, program.x, program.N, self.w_in, dt, None, False, "bottleneck.mid", "bottleneck.in")
        program.pending = emit_linear(program, mid.tensor(), program.N, self.w_out, dt, None, True, "bottleneck.out",
                                      "bottleneck.out")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_feed_forward_that_writes_its_own_launches(tmp_path, dtype):
    register_part("feed_forward", "bottleneck", BottleneckFeedForward, replace=True)
    H, nh, nkv, d, V, r = 80, 5, 5, 16, 90, 24

    @dataclass(frozen=True)
    class Toy8Config:
        model_type: str = "toy-bottleneck"

        @staticmethod
        def from_dict(raw, where="config.json"):
            return Toy8Config()

        def to_dict(self):
            return {"model_type": self.model_type}

    def spec(cfg):
        norm = lambda prefix: PartSpec("rmsnorm", {"size": H, "eps": 1e-6, "init": ("uniform", 0.5, 1.5)}, prefix)
        layers = [LayerSpec("prenorm",
                            PartSpec("attention", {"hidden_size": H, "num_heads": nh, "num_kv_heads": nkv, "head_dim": d,
                                                   "init_std": 0.15, "position": {"kind": "rope", "params": {
                                                       "head_dim": d, "theta": 1000.0}}}, f"l.{i}.attn."),
                            PartSpec("bottleneck", {"hidden_size": H, "rank": r}, f"l.{i}.ff."),
                            norm(f"l.{i}.n1."), norm(f"l.{i}.n2.")) for i in range(3)]
        return ModelSpec(vocab_size=V, hidden_size=H,
                         embedding=PartSpec("token", {"vocab_size": V, "hidden_size": H, "init_std": 0.5}, "emb."),
                         layers=layers, schedule=[ScheduleEntry(i) for i in range(3)], final_norm=norm("fn."),
                         head=PartSpec("linear", {"vocab_size": V, "hidden_size": H, "init_std": 0.1}, "head."))

    register_architecture("toy-bottleneck", Toy8Config, spec, replace=True)
    folder = write_random_model(Toy8Config(), str(tmp_path / "toy8"), seed=77,
                                dtype={"float32": torch.float32, "bfloat16": torch.bfloat16}[dtype])
    _, w = P.read_model(folder)

    def plain(ids):
        W = {k: v.double() for k, v in w.items()}
        T = len(ids)
        freqs, pos = 1000.0 ** (-torch.arange(0, d, 2, dtype=torch.float64) / d), torch.arange(T)
        h = P.embedding(W["emb.weight"], ids)
        for l in range(3):
            n = P.rms_norm(h, W[f"l.{l}.n1.weight"], 1e-6)
            p = f"l.{l}.attn."
            q = P.rope(P.linear(n, W[p + "q_proj.weight"]).reshape(T, nh, d), pos, freqs)
            k = P.rope(P.linear(n, W[p + "k_proj.weight"]).reshape(T, nkv, d), pos, freqs)
            v = P.linear(n, W[p + "v_proj.weight"]).reshape(T, nkv, d)
            h = h + P.linear(P.causal_attention(q, k, v, 1.0 / math.sqrt(d)).reshape(T, nh * d), W[p + "o_proj.weight"])
            m = P.rms_norm(h, W[f"l.{l}.n2.weight"], 1e-6)
            h = h + P.linear(P.linear(m, W[f"l.{l}.ff.in.weight"]), W[f"l.{l}.ff.out.weight"])
        return P.linear(P.rms_norm(h, W["fn.weight"], 1e-6), W["head.weight"])

    cache = lambda: CacheConfig(page_size=4, num_pages=48, num_state_slots=4, poison_freed_pages=True)
    eng = Engine.from_pretrained(folder, dtype=dtype, cache_config=cache())
    # the whole step is launched by the host library: no operation of the program is a call into Python
    assert eng.program is not None and eng.program.num_python_ops == 0 and eng.use_graphs
    twin = Engine.from_pretrained(folder, dtype=dtype, cache_config=cache(), executor="parts")
    assert twin.program is None
    reqs = TT.make_requests(V, (29, 7, 38, 18), seed=12)
    ref = {r_: plain(t) for r_, t in reqs.items()}
    tol = {"float32": 3e-5, "bfloat16": 8e-2}[dtype]
    for name, steps in (("whole", TT.trace_whole(reqs)), ("tail", TT.trace_tail_one_by_one(reqs, 12)),
                        ("portions", TT.trace_portions(reqs)),
                        ("mixed", TT.trace_mixed(reqs, {r_: max(2, len(t) - 8) for r_, t in reqs.items()}, seed=8)[0])):
        got = TT.run_steps(eng, steps)
        worst, rms, where = TT.error_against(got, ref)
        print(f"toy8 {dtype} {name}: {worst / rms:.2e} at {where}")
        assert worst == worst and worst <= tol * rms, (name, worst / rms, where)
        # the part's own launches make the bits of its forward
        by_parts = TT.run_steps(twin, steps)
        assert all(torch.equal(got[key], by_parts[key]) for key in got), name
    eng.program.check_guards()

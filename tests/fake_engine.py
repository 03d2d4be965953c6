"""A stand-in for the step function in tests of the scheduler and the generation loop
on the CPU: it keeps the engine's protocol with the cache manager (admit, reserve,
store) and returns "logits" that are a fixed function of the request's tokens so far,
so that what a request generates depends on its own history only, as with a model."""
import zlib

import numpy as np
import torch

from infernum_amd.cache import CacheConfig, CacheManager
from infernum_amd.engine import OutOfPages
from infernum_amd.parts import CacheSpec


def fake_logits(history, vocab):
    seed = zlib.crc32(np.asarray(history, dtype=np.int64).tobytes())
    return torch.from_numpy(np.random.RandomState(seed).standard_normal(vocab).astype(np.float32))


class FakeEngine:
    def __init__(self, vocab=50, page_size=4, num_pages=16, num_state_slots=8, needs=None):
        needs = needs or [(CacheSpec("full", 1, 16), None)]
        self.cache = CacheManager(needs, [None] * len(needs),
                                  CacheConfig(page_size=page_size, num_pages=num_pages,
                                              num_state_slots=num_state_slots), device=None)
        self.vocab = vocab
        self.history = {}
        self.steps = []            # per step: list of (request, number of tokens, wanted places)

    supports_device_tokens = True

    def step(self, entries, device_tokens=None, borrow_logits=False):
        """``device_tokens`` = (tokens of the last step, where the engine left them; per entry the place of its
        single token among them, or -1): as the real engine, which takes such tokens on the device."""
        rows = []
        log = []
        if device_tokens is not None:
            source, index = device_tokens
            entries = [type(e)(e.request, [int(source[j])], e.want) if j >= 0 else e for e, j in zip(entries, index)]
        for e in entries:
            need = self.cache.pages_needed(e.request, len(e.tokens))
            if any(n > g.allocator.num_free for n, g in zip(need, self.cache.groups)):
                raise OutOfPages(f"no pages for {e.request}")
            if not self.cache.has(e.request):
                assert self.cache.admit(e.request)
                self.history[e.request] = []
            assert self.cache.reserve(e.request, len(e.tokens))
            h = self.history[e.request]
            assert len(h) == self.cache.num_tokens(e.request)
            for j, t in enumerate(e.tokens):
                h.append(int(t))
                if j in e.want:
                    rows.append(fake_logits(h, self.vocab))
            self.cache.commit(e.request, len(e.tokens))
            log.append((e.request, len(e.tokens), list(e.want)))
        self.steps.append(log)
        self.cache.check()
        return torch.stack(rows) if rows else torch.empty((0, self.vocab))

    def end(self, request):
        if self.cache.has(request):
            self.cache.release(request)


class CpuSampler:
    """Greedy by argmax (first maximum); sampled rows by a plain inverse CDF of softmax(x / T)."""

    @staticmethod
    def needs_history(sampling):
        return False

    def select_on_device(self, logits, rows):
        return torch.tensor(self.select(logits, rows), dtype=torch.int32)

    def select(self, logits, rows):
        from infernum_amd.sampling import token_uniform
        out = []
        for x, r in zip(logits, rows):
            if r.sampling is None:
                out.append(int(torch.argmax(x)))
            else:
                p = torch.softmax(x.double() / r.sampling.temperature, 0)
                u = token_uniform(r.sampling.seed, r.generated_before)
                out.append(int(min(torch.searchsorted(torch.cumsum(p, 0), u * 0.999999), len(p) - 1)))
        return out


def reference_generation(prompt, options, vocab=50):
    """What a request generates when it runs alone and whole."""
    sampler = CpuSampler()
    from infernum_amd.sampling import RowRequest
    toks, out = list(prompt), []
    while len(out) < options.max_new_tokens:
        row = RowRequest(options.sampling, len(out), toks + out)
        t = sampler.select(fake_logits(toks + out, vocab)[None], [row])[0]
        if options.eos_token_id is not None and t == options.eos_token_id:
            break
        out.append(t)
    return out

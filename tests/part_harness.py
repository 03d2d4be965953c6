"""Runs single parts on the GPU in tests: a cache manager for the part's needs and
step contexts packed as the engine packs them."""
import torch

from infernum_amd.cache import CacheConfig, CacheManager
from infernum_amd.engine.batch import StepEntry, pack_step
from infernum_amd.parts import PartSpec, Runtime, make_part

DEV = torch.device("cuda:0")
DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}
# largest |difference| allowed as a fraction of the RMS of the plain result
TOL = {"float32": 2e-5, "bfloat16": 3e-2}


def runtime(dtype: str) -> Runtime:
    return Runtime(DEV, DTYPES[dtype])


def build(category, kind, params, rt, tensors=None, seed=0):
    """Make a part and give it weights: ``tensors`` (local name -> CPU tensor) or random ones."""
    part = make_part(category, PartSpec(kind, params), rt)
    g = torch.Generator().manual_seed(seed)
    given = {}
    for name, ws in part.weights().items():
        if tensors is not None and name in tensors:
            t = tensors[name].to(torch.float32)
        elif ws.init[0] == "normal":
            t = torch.randn(ws.shape, generator=g) * 0.3 / (ws.shape[-1] ** 0.5) * 4
        else:
            t = torch.rand(ws.shape, generator=g) + 0.5
        if rt.dtype == torch.bfloat16:
            t = t.to(torch.bfloat16).to(torch.float32)          # the plain side sees the values the part sees
        given[name] = t
    part.load({n: t.to(DEV).to(rt.dtype if part.weights()[n].follows_compute_dtype or rt.is_fp32 else t.dtype)
               for n, t in given.items()})
    return part, {n: t.double() for n, t in given.items()}


class Steps:
    """Contexts for one mixer (or a list of cache needs), step after step."""

    def __init__(self, needs, rt, page_size=4, num_pages=64, slots=8, poison=False):
        self.cache = CacheManager(needs, [None] * len(needs),
                                  CacheConfig(page_size=page_size, num_pages=num_pages, num_state_slots=slots,
                                              poison_freed_pages=poison), dtype=rt.dtype, device=DEV)
        self.views = self.cache.views()

    def begin(self, entries):
        """entries: (request, number of new tokens).  Returns (ctx, packed); call ``end`` after the part ran."""
        es = [StepEntry(r, [0] * n, []) for r, n in entries]
        for e in es:
            if not self.cache.has(e.request):
                assert self.cache.admit(e.request)
            assert self.cache.reserve(e.request, len(e.tokens))
        packed = pack_step(self.cache, es)
        return packed.context(torch.from_numpy(packed.host).to(DEV)), packed

    def end(self, packed):
        for e in packed.batch:
            self.cache.commit(e.request, len(e.tokens))


def rel_err(got: torch.Tensor, want: torch.Tensor) -> float:
    """Largest |difference| as a fraction of the RMS of the plain result.  A bf16 result is allowed,
    on top, the rounding of its own store (half a unit in the last of its 8 bits of mantissa, 2^-9 of the value)
    twice over: large values among small ones would otherwise set the measure."""
    want = want.double()
    d = (got.double().cpu() - want).abs()
    if got.dtype == torch.bfloat16:
        d = (d - want.abs() * 2.0 ** -8).clamp_min(0.0)
    return d.max().item() / max(want.pow(2).mean().sqrt().item(), 1e-30)


def dense(y, rt):
    """What a mixer or a feed-forward returned, as one tensor in the compute dtype."""
    from infernum_amd.kernels.api import SplitSum
    return y.joined(rt.dtype) if isinstance(y, SplitSum) else y

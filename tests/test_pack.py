"""The native packing of a step against a plain one written here: same arrays, same order of rows,
for random batches of prompt portions and single tokens over a full and a window group."""
import random

import numpy as np
import pytest

from infernum_amd.cache import NO_PAGE, CacheConfig, CacheManager, PageError
from infernum_amd.engine.batch import POW2_WIDTH, StepEntry, pack_step

PREFILL_TILE_ROWS = 64
from infernum_amd.parts import CacheSpec

FULL = CacheSpec("full", 2, 16)
WIN = CacheSpec("window", 2, 16, window=10)


def plain_pack(cache, entries, bt_width=None):
    """Rows: single tokens first, then the portions, each in the order given."""
    order = sorted(range(len(entries)), key=lambda i: (len(entries[i].tokens) != 1, i))
    batch = [entries[i] for i in order]
    q = [len(e.tokens) for e in batch]
    ctx = [cache.num_tokens(e.request) for e in batch]
    starts = [0]
    for n in q:
        starts.append(starts[-1] + n)
    row = {e.request: r for r, e in enumerate(batch)}
    out = {
        "token_ids": [t for e in batch for t in e.tokens],
        "positions": [c + j for c, n in zip(ctx, q) for j in range(n)],
        "token_seq": [r for r, n in enumerate(q) for _ in range(n)],
        "seq_starts": starts, "seq_ctx": ctx,
        "state_slots": [cache.state_slot(e.request) for e in batch],
        "logit_rows": [starts[row[e.request]] + w for e in entries for w in e.want],
    }
    # tiles of 64 queries of the portions, the ones with the most keys before them first
    tiles = [(r, q0) for r, n in enumerate(q) if n != 1 for q0 in range(0, n, PREFILL_TILE_ROWS)]
    tiles.sort(key=lambda t: -(ctx[t[0]] + t[1]))
    out["tiles"] = [v for t in tiles for v in t]
    ps = cache.page_size
    for g in range(len(cache.groups)):
        tables = [cache.block_table(g, e.request).pages for e in batch]
        width = bt_width or max(1, max(len(t) for t in tables))
        out[f"slots{g}"] = [t[p // ps] * ps + p % ps for t, c, n in zip(tables, ctx, q) for p in range(c, c + n)]
        out[f"bt{g}"] = [t[k] if k < len(t) else NO_PAGE for t in tables for k in range(width)]
        out[f"bt{g}_shape"] = (len(batch), width)
    return batch, q, ctx, out


def unpack(packed):
    seg = lambda i: packed.host[packed.offsets[i]:packed.offsets[i] + packed.sizes[i]].tolist()  # noqa: E731
    names = ["token_ids", "positions", "token_seq", "seq_starts", "seq_ctx", "state_slots", "logit_rows", "tiles"]
    out = {n: seg(i) for i, n in enumerate(names)}
    for g, shape in enumerate(packed.bt_shapes):
        out[f"slots{g}"], out[f"bt{g}"], out[f"bt{g}_shape"] = seg(8 + 2 * g), seg(9 + 2 * g), tuple(shape)
    return out


@pytest.mark.parametrize("seed", range(8))
def test_native_packing_equals_plain_packing(seed):
    rng = random.Random(seed)
    needs = [(FULL, None), (WIN, None)] if seed % 2 else [(FULL, None)]
    cache = CacheManager(needs, [None] * len(needs),
                         CacheConfig(page_size=rng.choice((2, 4, 16)), num_pages=4000, num_state_slots=6), device=None)
    live = {}
    for step in range(40):
        entries = []
        for r in list(live):
            if rng.random() < 0.7:
                n = 1 if rng.random() < 0.6 else rng.choice((2, 3, 9, 70, 130))
                entries.append(StepEntry(r, [rng.randrange(1000) for _ in range(n)],
                                         sorted(rng.sample(range(n), rng.randint(0, min(n, 3))))))
        if len(live) < 5 and rng.random() < 0.5:
            r = f"req{step}"
            n = rng.choice((1, 2, 5, 64, 65, 200))
            assert cache.admit(r)
            live[r] = 0
            entries.append(StepEntry(r, [rng.randrange(1000) for _ in range(n)], [n - 1]))
        rng.shuffle(entries)
        if not entries:
            continue
        for e in entries:
            assert cache.reserve(e.request, len(e.tokens))
        width = None
        if all(len(e.tokens) == 1 for e in entries) and rng.random() < 0.5:
            width = 8
            while width < max(len(cache.block_table(g, e.request).pages) for g in range(len(needs)) for e in entries):
                width *= 2
        # the native side finds that power of two itself when asked to
        packed = pack_step(cache, entries, bt_width=POW2_WIDTH if width and step % 2 else width, tile_rows=PREFILL_TILE_ROWS)
        batch, q, ctx, want = plain_pack(cache, entries, width)
        assert [e.request for e in packed.batch] == [e.request for e in batch]
        assert packed.q_lens == q and packed.ctx_lens == ctx
        assert packed.num_decode == sum(1 for n in q if n == 1)
        assert packed.num_tiles == len(want["tiles"]) // 2 and packed.num_logit_rows == len(want["logit_rows"])
        assert unpack(packed) == want
        assert all(o % 4 == 0 for o in packed.offsets) and packed.host.dtype == np.int32
        for e in entries:
            cache.commit(e.request, len(e.tokens))
            live[e.request] += len(e.tokens)
        for r in list(live):
            if live[r] > 300 or rng.random() < 0.05:
                cache.release(r)
                del live[r]
        cache.check()


def test_packing_refuses_tokens_without_pages_and_unknown_requests():
    cache = CacheManager([(FULL, None)], [None], CacheConfig(page_size=4, num_pages=8, num_state_slots=2), device=None)
    cache.admit("a")
    with pytest.raises(PageError, match="no page"):
        pack_step(cache, [StepEntry("a", [1, 2, 3], [2])])
    with pytest.raises(PageError, match="not admitted"):
        pack_step(cache, [StepEntry("b", [1], [0])])
    assert cache.reserve("a", 20)
    with pytest.raises(PageError, match="wider"):
        pack_step(cache, [StepEntry("a", [1] * 20, [])], bt_width=2)

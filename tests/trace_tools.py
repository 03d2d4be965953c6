"""Builders of replay traces (lists of steps) for the equivalence tests, and the
comparison of what a replay returns with the plain implementation."""
import random
from typing import Dict, List, Sequence, Tuple

import torch


def make_requests(vocab: int, lengths: Sequence[int], seed: int) -> Dict[str, List[int]]:
    rng = random.Random(seed)
    return {f"r{i}": [rng.randrange(vocab) for _ in range(n)] for i, n in enumerate(lengths)}


def _step(i, entries, end=()):
    return {"step": i, "entries": [{"id": r, "tokens": list(t), "want": list(w)} for r, t, w in entries],
            "end": list(end)}


def trace_whole(reqs) -> List[dict]:
    """Each request alone and whole: one step, every place wanted."""
    return [_step(i, [(r, toks, range(len(toks)))], [r]) for i, (r, toks) in enumerate(reqs.items())]


def trace_tail_one_by_one(reqs, tail: int = 32) -> List[dict]:
    """Most of a request in one step, its last ``tail`` tokens one by one."""
    steps = []
    for r, toks in reqs.items():
        head = max(1, len(toks) - tail)
        steps.append(_step(len(steps), [(r, toks[:head], range(head))]))
        for p in range(head, len(toks)):
            steps.append(_step(len(steps), [(r, toks[p:p + 1], [0])], [r] if p == len(toks) - 1 else []))
        if head == len(toks):
            steps[-1]["end"] = [r]
    return steps


def trace_portions(reqs, sizes=(8, 5, 3, 2, 2, 7, 13, 2, 31, 4)) -> List[dict]:
    """One request at a time in portions of changing size, down to two tokens."""
    steps = []
    for r, toks in reqs.items():
        p, k = 0, 0
        while p < len(toks):
            n = min(sizes[k % len(sizes)], len(toks) - p)
            if len(toks) - p - n == 1:      # leave no single token: the last portion takes it
                n += 1
            k += 1
            last = p + n == len(toks)
            steps.append(_step(len(steps), [(r, toks[p:p + n], range(n))], [r] if last else []))
            p += n
    return steps


def trace_mixed(reqs, prompt_len: Dict[str, int], seed: int = 0, max_live: int = 4) -> Tuple[List[dict], int]:
    """Up to ``max_live`` live requests; portions of prompts of some beside single
    decoded tokens of others; requests pause now and then; a finished request's
    place is taken by the next.  Returns (steps, max_tokens): the most tokens live
    requests hold at any time, each rounded up to 64, so that a pool of exactly
    that size makes later requests reuse the pages of earlier ones."""
    rng = random.Random(seed)
    waiting = list(reqs.keys())
    live: List[str] = []
    fed: Dict[str, int] = {}
    steps: List[dict] = []
    max_tokens = 0
    while waiting or live:
        while waiting and len(live) < max_live and (not live or rng.random() < 0.6):
            r = waiting.pop(0)
            live.append(r)
            fed[r] = 0
        entries, ended = [], []
        for r in list(live):
            if len(live) > 1 and rng.random() < 0.15:
                continue                                    # left out of this step, goes on later
            toks, p = reqs[r], fed[r]
            if p < prompt_len[r]:
                n = min(rng.choice((2, 3, 5, 8, 13, 21)), prompt_len[r] - p)
                if prompt_len[r] - p - n == 1:
                    n += 1
            else:
                n = 1
            n = min(n, len(toks) - p)
            entries.append((r, toks[p:p + n], range(n)))
            fed[r] = p + n
            if fed[r] == len(toks):
                ended.append(r)
        if not entries:
            continue
        held = sum(-(-fed[r] // 64) * 64 for r in live)
        max_tokens = max(max_tokens, held)
        steps.append(_step(len(steps), entries, ended))
        for r in ended:
            live.remove(r)
    return steps, max_tokens


def run_steps(engine, steps) -> Dict[Tuple[str, int], torch.Tensor]:
    """Replay steps through an Engine; (request, position) -> logits row (CPU fp32)."""
    from infernum_amd.engine import StepEntry
    pos: Dict[str, int] = {}
    out: Dict[Tuple[str, int], torch.Tensor] = {}
    for s in steps:
        entries = [StepEntry(e["id"], e["tokens"], e["want"]) for e in s["entries"]]
        logits = engine.step(entries).to("cpu")
        row = 0
        for e in s["entries"]:
            base = pos.get(e["id"], 0)
            for w in e["want"]:
                out[(e["id"], base + w)] = logits[row]
                row += 1
            pos[e["id"]] = base + len(e["tokens"])
        assert row == logits.shape[0]
        for r in s["end"]:
            engine.end(r)
            pos.pop(r, None)
    return out


def error_against(got: Dict[Tuple[str, int], torch.Tensor], want: Dict[str, torch.Tensor], every_place: bool = True):
    """Largest |difference| over all rows, the RMS of the wanted logits, and where the largest is.
    ``every_place``: the replay must have returned a row for every place of every request of ``want``
    (the traces of this file want them all), so that a row that never came back cannot pass."""
    if every_place:
        missing = [(r, p) for r, ref in want.items() for p in range(ref.shape[0]) if (r, p) not in got]
        assert not missing, f"{len(missing)} places have no logits, the first {missing[:5]}"
        assert len(got) == sum(ref.shape[0] for ref in want.values()), "rows for places that no request has"
    worst, where = 0.0, None
    sq, n = 0.0, 0
    for (r, p), row in got.items():
        ref = want[r][p].to(torch.float64)
        d = (row.to(torch.float64) - ref).abs().max().item()
        if not (d == d):
            return float("nan"), 1.0, (r, p)
        if d > worst:
            worst, where = d, (r, p)
        sq += float((ref * ref).sum())
        n += ref.numel()
    return worst, (sq / max(n, 1)) ** 0.5, where


def rms_error_against(got: Dict[Tuple[str, int], torch.Tensor], want: Dict[str, torch.Tensor]) -> float:
    """Root mean square of the difference over all rows, as a fraction of the RMS of the wanted logits: where the
    largest difference is set by one unlucky logit among millions, this one tells what the rows are like."""
    sq_d, sq_w, n = 0.0, 0.0, 0
    for (r, p), row in got.items():
        ref = want[r][p].to(torch.float64)
        sq_d += float((row.to(torch.float64) - ref).pow(2).sum())
        sq_w += float((ref * ref).sum())
        n += ref.numel()
    return (sq_d / max(sq_w, 1e-300)) ** 0.5

"""Iteration-level scheduling of requests over the step function.

Requests wait in a queue and are admitted first come, first served, without
skipping a request that does not fit (infernum-runtime/src/scheduler.rs:318-338).
Every step holds, in this order: one token of every running request that is
decoding (scheduler.rs:311-315), the next portions of the prompts of running
requests, then first portions of newly admitted ones; all under one budget of
tokens per step, a portion being at most ``max_prefill_tokens`` long.  The
reference gives every admitted request its own full chunk in the same iteration
and never schedules later chunks (``continue_prefill`` has no caller but its
test, scheduler.rs:363-381); here a prompt's portions follow each other step by
step until it is done.  Pages are taken for the tokens of a step only, not for a
whole prompt at admission.

When pages run out: a decoding request that needs a page which the pool cannot
give sets back the request that was admitted last (possibly itself): that
request gives all its pages and its state slot back and returns to the front of
the queue with what it has generated so far appended to its prompt, to be
computed again later.  What a request generates does not change by that: its
tokens depend on its own history only (sampling draws are keyed by the seed and
the number of tokens generated so far).  A portion of a prompt is cut down to the
pages that are free; when no request at all can move, the last admitted request
is set back in the same way.  A request that is alone and still cannot get its
pages ends with an error: the pool is too small for it.  (The reference stops
admitting when blocks run out, scheduler.rs:327-330, never sets a request back,
and ignores a failed allocation while decoding, engine.rs:476-480.)

The scheduler only decides; it keeps no tensors and calls no kernels.  It reads
the cache manager's counts, and gives back what finished or set-back requests
hold.
"""
from __future__ import annotations

import enum
from collections import deque
from dataclasses import dataclass, field
from typing import Callable, Deque, Hashable, List, Optional, Sequence

from ..cache import CacheManager
from ..sampling.params import GenerateOptions


class FinishReason(enum.Enum):
    """Why a generation ended (scheduler.rs:23-31)."""

    STOP = "stop"              # the end-of-sequence token came (it is not emitted)
    LENGTH = "length"          # max_new_tokens (or the longest allowed sequence) was reached
    CANCELLED = "cancelled"    # the receiver went away


@dataclass
class GenerationEvent:
    """Zero or more ``token`` events, then exactly one ``finished`` or ``error`` (scheduler.rs:37-44)."""

    kind: str                                  # "token" | "finished" | "error"
    token: Optional[int] = None
    reason: Optional[FinishReason] = None
    error: Optional[str] = None


TokenSender = Callable[[GenerationEvent], bool]     # returns False when nobody listens any more


@dataclass
class BatchConfig:
    """The reference's four settings with its defaults (scheduler.rs:73-95) and the
    budget of tokens per step, which the reference does not have."""

    max_batch_size: int = 32          # most requests running at once
    max_prefill_tokens: int = 512     # longest portion of one prompt in one step
    block_size: int = 16              # tokens per page
    num_blocks: int = 1024            # pages in the pool
    max_tokens_per_step: int = 2048   # all tokens of one step, decoded ones included

    def __post_init__(self) -> None:
        for name in ("max_batch_size", "max_prefill_tokens", "block_size", "num_blocks", "max_tokens_per_step"):
            if int(getattr(self, name)) <= 0:
                raise ValueError(f"{name} must be positive")
        if self.max_tokens_per_step < self.max_batch_size:
            raise ValueError("max_tokens_per_step must be at least max_batch_size: every running request decodes "
                             "one token per step")


class SequencePhase(enum.Enum):
    WAITING = "waiting"
    PREFILL = "prefill"
    DECODE = "decode"
    FINISHED = "finished"


@dataclass(eq=False)
class SequenceState:
    """What the scheduler knows of one request (scheduler.rs:111-163)."""

    id: Hashable
    prompt_ids: List[int]
    options: GenerateOptions
    token_tx: Optional[TokenSender] = None
    generated_ids: List[int] = field(default_factory=list)
    phase: SequencePhase = SequencePhase.WAITING
    finish_reason: Optional[FinishReason] = None
    error: Optional[str] = None
    times_set_back: int = 0

    def all_tokens(self) -> List[int]:
        return self.prompt_ids + self.generated_ids

    @property
    def num_tokens(self) -> int:
        return len(self.prompt_ids) + len(self.generated_ids)

    def send(self, event: GenerationEvent) -> bool:
        return True if self.token_tx is None else bool(self.token_tx(event))


@dataclass
class PrefillTask:
    """A portion of a request's tokens; ``completes`` when it reaches the request's last token."""

    seq: SequenceState
    token_ids: List[int]
    completes: bool


@dataclass
class DecodeTask:
    seq: SequenceState


@dataclass
class SchedulerOutput:
    decode: List[DecodeTask] = field(default_factory=list)
    prefill: List[PrefillTask] = field(default_factory=list)
    set_back: List[SequenceState] = field(default_factory=list)
    finished: List[SequenceState] = field(default_factory=list)    # reaped in this step

    @property
    def num_tokens(self) -> int:
        return len(self.decode) + sum(len(t.token_ids) for t in self.prefill)

    def is_empty(self) -> bool:
        return not self.decode and not self.prefill


class Scheduler:
    def __init__(self, config: BatchConfig, max_seq_len: Optional[int] = None):
        self.config = config
        self.max_seq_len = max_seq_len
        self.waiting: Deque[SequenceState] = deque()
        self.running: List[SequenceState] = []        # in the order of admission
        self._next_id = 0

    # ---- requests ---------------------------------------------------------------
    def add_request(self, prompt_ids: Sequence[int], options: GenerateOptions,
                    token_tx: Optional[TokenSender] = None) -> SequenceState:
        prompt = [int(t) for t in prompt_ids]
        if not prompt:
            raise ValueError("a request needs at least one prompt token")
        if self.max_seq_len is not None and len(prompt) > self.max_seq_len:
            raise ValueError(f"prompt of {len(prompt)} tokens is longer than max_seq_len {self.max_seq_len}")
        seq = SequenceState(self._next_id, prompt, options, token_tx)
        self._next_id += 1
        if options.max_new_tokens == 0:
            self._finish(seq, FinishReason.LENGTH)
            return seq
        self.waiting.append(seq)
        return seq

    def is_idle(self) -> bool:
        return not self.waiting and not self.running

    def num_running(self) -> int:
        return len(self.running)

    def num_waiting(self) -> int:
        return len(self.waiting)

    def reap(self, cache: CacheManager) -> List[SequenceState]:
        """Finished requests leave the running list and give back what they hold."""
        done = [s for s in self.running if s.phase == SequencePhase.FINISHED]
        for seq in done:
            self.running.remove(seq)
            if cache.has(seq.id):
                cache.release(seq.id)
        return done

    # ---- one step -----------------------------------------------------------------
    def step(self, cache: CacheManager) -> SchedulerOutput:
        cfg = self.config
        out = SchedulerOutput()
        # 1. finished requests give back what they hold (scheduler.rs:289-305)
        out.finished.extend(self.reap(cache))

        budget = cfg.max_tokens_per_step
        promised = [0] * len(cache.groups)        # pages this step's earlier entries will take
        new_slots = 0

        def fits(need: List[int]) -> bool:
            return all(n + p <= g.allocator.num_free for n, p, g in zip(need, promised, cache.groups))

        def take(need: List[int]) -> None:
            for i, n in enumerate(need):
                promised[i] += n

        # 2. one token for every decoding request
        i = 0
        while i < len(self.running):
            seq = self.running[i]
            if seq.phase != SequencePhase.DECODE:
                i += 1
                continue
            need = cache.pages_needed(seq.id, 1)
            if fits(need):
                take(need)
                budget -= 1
                out.decode.append(DecodeTask(seq))
                i += 1
                continue
            victim = self.running[-1]
            if victim is seq and len(self.running) == 1:
                self._fail(seq, f"the page pool is too small for a request of {seq.num_tokens + 1} tokens")
                self.running.remove(seq)
                cache.release(seq.id)
                out.finished.append(seq)
                continue
            self._set_back(victim, cache, out)
            # the victim stood at or after i: position i now holds the next request (or none)

        # 3. next portions of running prompts, in the order of admission
        blocked = False
        i = 0
        while i < len(self.running):
            seq = self.running[i]
            if seq.phase != SequencePhase.PREFILL:
                i += 1
                continue
            if budget <= 0:
                break
            cached = cache.num_tokens(seq.id) if cache.has(seq.id) else 0
            n = min(seq.num_tokens - cached, cfg.max_prefill_tokens, budget)
            n = min(n, cache.tokens_that_fit(seq.id, promised) if cache.has(seq.id)
                    else cache.tokens_that_fit(None, promised))
            if n <= 0:
                if out.is_empty():
                    # nobody can move: the last admitted request makes room
                    victim = self.running[-1]
                    if victim is seq and len(self.running) == 1:
                        self._fail(seq, f"the page pool is too small for a request of {seq.num_tokens} tokens")
                        self.running.remove(seq)
                        if cache.has(seq.id):
                            cache.release(seq.id)
                        out.finished.append(seq)
                        continue
                    self._set_back(victim, cache, out)
                    continue
                blocked = True
                break
            if not cache.has(seq.id):
                new_slots += 1
            take(cache.pages_needed(seq.id, n))
            budget -= n
            tokens = seq.all_tokens()[cached:cached + n]
            out.prefill.append(PrefillTask(seq, tokens, cached + n == seq.num_tokens))
            i += 1

        # 4. admissions, first come first served, while the head of the queue fits
        while (self.waiting and not blocked and not out.set_back and budget > 0
               and len(self.running) < cfg.max_batch_size and cache.slots.num_free - new_slots > 0):
            seq = self.waiting[0]
            n = min(seq.num_tokens, cfg.max_prefill_tokens, budget)
            need = cache.pages_needed(seq.id, n)
            # keep one page in hand for every running request, so that a newcomer is not set back at once
            spare = [len(self.running)] * len(need) if self.running else [0] * len(need)
            if not fits([a + b for a, b in zip(need, spare)]):
                if not self.running and out.is_empty():
                    # alone and still too large for one portion: shrink the portion to the pool
                    n = min(n, cache.tokens_that_fit(None, promised))
                    if n <= 0:
                        self.waiting.popleft()
                        self._fail(seq, "the page pool has no free page although nothing is running")
                        out.finished.append(seq)
                        continue
                    need = cache.pages_needed(seq.id, n)
                else:
                    break
            self.waiting.popleft()
            seq.phase = SequencePhase.PREFILL
            self.running.append(seq)
            new_slots += 1
            take(need)
            budget -= n
            out.prefill.append(PrefillTask(seq, seq.all_tokens()[:n], n == seq.num_tokens))
        return out

    # ---- after the model has run ------------------------------------------------------
    def on_prefill_done(self, task: PrefillTask, token: Optional[int]) -> None:
        """The portion is in the cache; ``token`` is the one chosen after a portion that completes."""
        if task.seq.phase == SequencePhase.FINISHED:
            return
        if task.completes:
            if token is None:
                raise ValueError("a completed prompt needs its next token")
            task.seq.phase = SequencePhase.DECODE
            self.handle_new_token(task.seq, token)

    def on_decode_done(self, task: DecodeTask, token: int) -> None:
        if task.seq.phase != SequencePhase.FINISHED:
            self.handle_new_token(task.seq, token)

    def handle_new_token(self, seq: SequenceState, token: int) -> None:
        """infernum-runtime/src/engine.rs:445-481: the end-of-sequence token stops and is
        not emitted; a receiver that went away cancels; max_new_tokens ends with LENGTH."""
        token = int(token)
        if seq.options.eos_token_id is not None and token == seq.options.eos_token_id:
            self._finish(seq, FinishReason.STOP)
            return
        seq.generated_ids.append(token)
        if not seq.send(GenerationEvent("token", token=token)):
            seq.phase = SequencePhase.FINISHED
            seq.finish_reason = FinishReason.CANCELLED
            return
        if len(seq.generated_ids) >= seq.options.max_new_tokens:
            self._finish(seq, FinishReason.LENGTH)
        elif self.max_seq_len is not None and seq.num_tokens >= self.max_seq_len:
            self._finish(seq, FinishReason.LENGTH)

    def cancel(self, seq: SequenceState) -> None:
        """The caller does not want the rest; what the request holds goes back at the next step."""
        if seq.phase == SequencePhase.FINISHED:
            return
        if seq.phase == SequencePhase.WAITING:
            self.waiting.remove(seq)
        seq.phase = SequencePhase.FINISHED
        seq.finish_reason = FinishReason.CANCELLED

    # ---- helpers ------------------------------------------------------------------------
    def _finish(self, seq: SequenceState, reason: FinishReason) -> None:
        seq.phase = SequencePhase.FINISHED
        seq.finish_reason = reason
        seq.send(GenerationEvent("finished", reason=reason))

    def _fail(self, seq: SequenceState, message: str) -> None:
        seq.phase = SequencePhase.FINISHED
        seq.error = message
        seq.send(GenerationEvent("error", error=message))

    def _set_back(self, victim: SequenceState, cache: CacheManager, out: SchedulerOutput) -> None:
        self.running.remove(victim)
        if cache.has(victim.id):
            cache.release(victim.id)
        # drop what this step had planned for it
        out.decode = [t for t in out.decode if t.seq is not victim]
        out.prefill = [t for t in out.prefill if t.seq is not victim]
        victim.phase = SequencePhase.WAITING
        victim.times_set_back += 1
        self.waiting.appendleft(victim)
        out.set_back.append(victim)

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
hold.  The decisions of a step are taken natively (``ia_sched_step`` in
csrc/host_core.cpp, beside the cache's bookkeeping); this module keeps the
requests themselves, their tokens, phases and events, and applies the decisions.
"""
from __future__ import annotations

import ctypes
import enum
from collections import deque
from dataclasses import dataclass, field
from typing import Callable, Deque, Hashable, List, Optional, Sequence

from ..cache import CacheManager, native
from ..sampling.params import GenerateOptions

_ACT_DECODE, _ACT_PORTION, _ACT_SET_BACK, _ACT_FAIL, _ACT_ADMIT = 1, 2, 3, 4, 5     # kinds of ia_sched_step's actions


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
    # A portion that does not reach its prompt's end stops where the step's tokens are a multiple of this, if that
    # leaves it at least half of what it could take: the library's products work in tiles of 256 rows (8,200 rows
    # take what 8,448 do, a third to half more than 8,192), so a portion beside decoded tokens leaves them their rows.
    # 1: portions are cut by the other limits alone, as the reference cuts them.
    step_token_multiple: int = 256

    def __post_init__(self) -> None:
        for name in ("max_batch_size", "max_prefill_tokens", "block_size", "num_blocks", "max_tokens_per_step",
                     "step_token_multiple"):
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
    pending: int = 0            # tokens chosen on the device in a step whose result the host has not seen yet

    def all_tokens(self) -> List[int]:
        """The tokens the host knows (a pending one is not among them)."""
        return self.prompt_ids + self.generated_ids

    @property
    def num_tokens(self) -> int:
        return len(self.prompt_ids) + len(self.generated_ids) + self.pending

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
        """The decisions themselves are taken natively (``ia_sched_step`` in csrc/host_core.cpp) over the
        cache's counts; here they are applied to the requests."""
        cfg = self.config
        out = SchedulerOutput()
        # finished requests give back what they hold (scheduler.rs:289-305)
        out.finished.extend(self.reap(cache))
        running, waiting = list(self.running), list(self.waiting)
        if not running and not waiting:
            return out
        nr, nw = len(running), len(waiting)
        rid = (ctypes.c_int64 * max(nr, 1))(*[cache.request_id(s.id) if cache.has(s.id) else -1 for s in running])
        # 3: a request whose last token is still on the device keeps what it holds and does nothing more
        phase = (ctypes.c_int * max(nr, 1))(*[3 if self._awaits_last_token(s) else
                                              (2 if s.phase == SequencePhase.DECODE else 1) for s in running])
        tokens = (ctypes.c_int64 * max(nr, 1))(*[s.num_tokens for s in running])
        wait_tokens = (ctypes.c_int64 * max(nw, 1))(*[s.num_tokens for s in waiting])
        cap = 3 * nr + 2 * nw + 4
        actions = (ctypes.c_int * (4 * cap))()
        n = native.lib().ia_sched_step(cache.native_handle(), nr, rid, phase, tokens, nw, wait_tokens,
                                       cfg.max_batch_size, cfg.max_prefill_tokens, cfg.max_tokens_per_step,
                                       cfg.step_token_multiple, actions, cap)
        if n < 0:
            cache._fail()
        cache.poison_freed()
        for i in range(n):
            kind, index, a, b = actions[4 * i:4 * i + 4]
            if kind == _ACT_DECODE:
                out.decode.append(DecodeTask(running[index]))
            elif kind == _ACT_PORTION:
                seq = running[index]
                out.prefill.append(PrefillTask(seq, seq.all_tokens()[a:a + b], a + b == seq.num_tokens))
            elif kind == _ACT_SET_BACK:
                seq = running[index]
                self.running.remove(seq)
                cache.forget(seq.id)                       # released natively while deciding
                seq.phase = SequencePhase.WAITING
                seq.times_set_back += 1
                self.waiting.appendleft(seq)
                out.set_back.append(seq)
            elif kind == _ACT_FAIL and a == 3:
                seq = self._pop_waiting(waiting[index])
                self._fail(seq, "the page pool has no free page although nothing is running")
                out.finished.append(seq)
            elif kind == _ACT_FAIL:
                seq = running[index]
                size = seq.num_tokens + 1 if a == 1 else seq.num_tokens
                self._fail(seq, f"the page pool is too small for a request of {size} tokens")
                self.running.remove(seq)
                cache.forget(seq.id)
                out.finished.append(seq)
            elif kind == _ACT_ADMIT:
                seq = self._pop_waiting(waiting[index])
                seq.phase = SequencePhase.PREFILL
                self.running.append(seq)
                out.prefill.append(PrefillTask(seq, seq.all_tokens()[:b], b == seq.num_tokens))
            else:
                raise RuntimeError(f"unknown scheduling action {kind}")
        return out

    def _awaits_last_token(self, seq: SequenceState) -> bool:
        if not seq.pending or seq.phase == SequencePhase.FINISHED:
            return False
        return (len(seq.generated_ids) + seq.pending >= seq.options.max_new_tokens
                or (self.max_seq_len is not None and seq.num_tokens >= self.max_seq_len))

    # ---- while the model runs: the step is launched, its tokens are not here yet ------
    def on_launched(self, plan: SchedulerOutput) -> None:
        """The step of ``plan`` was launched and leaves its chosen tokens on the device: every request that gets
        a token from it counts one token more from now on; ``on_decode_done`` / ``on_prefill_done`` bring it."""
        for t in plan.decode:
            t.seq.pending += 1
        for t in plan.prefill:
            if t.completes:
                t.seq.phase = SequencePhase.DECODE
                t.seq.pending += 1

    # ---- after the model has run ------------------------------------------------------
    def on_prefill_done(self, task: PrefillTask, token: Optional[int]) -> None:
        """The portion is in the cache; ``token`` is the one chosen after a portion that completes."""
        if task.completes:
            if token is None:
                raise ValueError("a completed prompt needs its next token")
            if task.seq.phase == SequencePhase.PREFILL:
                task.seq.phase = SequencePhase.DECODE
            self.handle_new_token(task.seq, token)

    def on_decode_done(self, task: DecodeTask, token: int) -> None:
        self.handle_new_token(task.seq, token)

    def handle_new_token(self, seq: SequenceState, token: int) -> None:
        """infernum-runtime/src/engine.rs:445-481: the end-of-sequence token stops and is
        not emitted; a receiver that went away cancels; max_new_tokens ends with LENGTH."""
        token = int(token)
        if seq.pending:
            seq.pending -= 1                      # the token that was on the device
        if seq.phase == SequencePhase.FINISHED:
            return
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
    def _pop_waiting(self, expected: SequenceState) -> SequenceState:
        seq = self.waiting.popleft()
        if seq is not expected:
            raise RuntimeError("the queue changed while a step was decided")
        return seq

    def _finish(self, seq: SequenceState, reason: FinishReason) -> None:
        if seq.phase == SequencePhase.WAITING and seq in self.waiting:
            self.waiting.remove(seq)              # set back while its last token was still on the device
        seq.phase = SequencePhase.FINISHED
        seq.finish_reason = reason
        seq.send(GenerationEvent("finished", reason=reason))

    def _fail(self, seq: SequenceState, message: str) -> None:
        seq.phase = SequencePhase.FINISHED
        seq.error = message
        seq.send(GenerationEvent("error", error=message))

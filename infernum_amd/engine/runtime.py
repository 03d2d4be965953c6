"""The generation loop: scheduler, step function and sampler put together.

``Runtime`` is what a user of the package talks to.  It takes requests
(``submit``), and every ``step`` asks the scheduler for a batch, runs it through
:meth:`Engine.step` as one mixed batch, chooses the next token of every request
whose last token was in the batch, and tells the scheduler.  ``generate`` and
``generate_stream`` drive the loop until their request is done; any other
requests that are waiting or running move along in the same steps.

The reference splits this over ``Engine`` (a worker thread fed through a
channel, infernum-runtime/src/engine.rs:39-238) and ``Runtime`` (tokenizer on
top, infernum-runtime/src/runtime.rs:17-135).  Here one object runs on the
caller's thread: the model, the cache and the scheduler have one owner, and
nothing needs a lock.
"""
from __future__ import annotations

import os
from typing import Any, Callable, Iterator, List, Optional, Sequence, Union

from ..cache import CacheConfig
from ..sampling.params import GenerateOptions
from ..sampling.sampler import RowRequest
from .engine import Engine, StepEntry
from .scheduler import BatchConfig, Scheduler, SchedulerOutput, SequencePhase, SequenceState, TokenSender

Prompt = Union[str, Sequence[int]]


class GenerationError(RuntimeError):
    pass


class _TokensAtHand:
    """The tokens of an engine that keeps them where the host reads them anyway (stand-ins on the CPU)."""

    @staticmethod
    def start(tokens):
        return tokens

    @staticmethod
    def wait(handle) -> List[int]:
        return [int(t) for t in handle.tolist()]


class Runtime:
    def __init__(self, engine: Any, tokenizer: Any = None, batch_config: Optional[BatchConfig] = None,
                 max_seq_len: Optional[int] = None, sampler: Any = None):
        """``engine`` has ``step(entries)``, ``end(request)`` and ``cache``; ``sampler`` has
        ``select(logits, rows)``; ``tokenizer`` (optional) has ``encode`` and ``decode``."""
        self.engine = engine
        self.tokenizer = tokenizer
        cc = engine.cache.config
        if batch_config is None:
            batch_config = BatchConfig(block_size=cc.page_size, num_blocks=cc.num_pages,
                                       max_batch_size=min(32, cc.num_state_slots))
        if batch_config.block_size != cc.page_size or batch_config.num_blocks != cc.num_pages:
            raise ValueError("batch_config's block_size and num_blocks must be those the engine's cache was made with")
        if batch_config.max_batch_size > cc.num_state_slots:
            raise ValueError("max_batch_size is larger than the number of state slots of the cache")
        limit = getattr(getattr(engine, "rt", None), "max_tokens_per_step", None)
        if limit is not None and batch_config.max_tokens_per_step > limit:
            raise ValueError(f"max_tokens_per_step {batch_config.max_tokens_per_step} is above the engine's {limit}")
        self.batch_config = batch_config
        if max_seq_len is None:
            # the model's own bound (max_position_embeddings; infernum-llama/src/config.rs:44-45, ModelConfig.max_seq_len)
            max_seq_len = getattr(getattr(engine, "spec", None), "max_position", 0) or None
        self.scheduler = Scheduler(batch_config, max_seq_len=max_seq_len)
        if sampler is None:
            from ..sampling.sampler import Sampler
            sampler = Sampler(engine.rt.device)
        self.sampler = sampler
        self.steps = 0
        self.tokens_run = 0
        # One step ahead: a step is launched with the tokens of the step before it still on the device, and the
        # host reads a step's tokens while the next step runs.  Needs an engine that takes tokens from the device
        # and a sampler that leaves them there; a choice that looks at the request's own last tokens (a repetition
        # penalty) finds the newest of them on the device too, with a sampler that says so (``history_on_device``;
        # with another, such requests are served one step at a time).
        self.look_ahead = (getattr(engine, "supports_device_tokens", False)
                           and hasattr(self.sampler, "select_on_device") and hasattr(self.sampler, "needs_history"))
        self._inflight = None                 # (plan, tokens on the device, row of each request, download)
        self._download = None
        self._recomputed = 0                  # requests served without the cache so far (their names)

    # ---- building ---------------------------------------------------------------------
    @classmethod
    def from_pretrained(cls, model_dir: str, dtype: Any = "bfloat16", batch_config: Optional[BatchConfig] = None,
                        max_seq_len: Optional[int] = None, device: Any = "cuda:0", kernels: str = "auto") -> "Runtime":
        bc = batch_config or BatchConfig()
        engine = Engine.from_pretrained(
            model_dir, dtype=dtype, device=device, max_tokens_per_step=bc.max_tokens_per_step, kernels=kernels,
            cache_config=CacheConfig(page_size=bc.block_size, num_pages=bc.num_blocks,
                                     num_state_slots=bc.max_batch_size))
        return cls(engine, load_tokenizer(model_dir), bc, max_seq_len)

    # ---- requests ----------------------------------------------------------------------
    def submit(self, input_ids: Sequence[int], options: GenerateOptions,
               token_tx: Optional[TokenSender] = None) -> SequenceState:
        """Queue a request; its tokens arrive through ``token_tx`` as the loop runs (engine.rs:112-126)."""
        V = getattr(getattr(self.engine, "spec", None), "vocab_size", None)
        if V is not None and any(not 0 <= int(t) < V for t in input_ids):
            raise ValueError(f"prompt holds a token id outside the vocabulary [0, {V})")
        return self.scheduler.add_request(input_ids, options, token_tx)

    def step(self) -> SchedulerOutput:
        """One iteration: schedule, run the batch, choose tokens, update (engine.rs:191-237).  With look-ahead
        the tokens of the step launched here reach the requests during the next call."""
        if self.look_ahead and self._all_can_wait():
            return self._step_ahead()
        self._deliver()
        plan = self.scheduler.step(self.engine.cache)
        if plan.is_empty():
            return plan
        entries: List[StepEntry] = []
        rows: List[RowRequest] = []
        for t in plan.decode:
            s = t.seq
            entries.append(StepEntry(s.id, [s.generated_ids[-1]], [0]))
            rows.append(self._row(s))
        for t in plan.prefill:
            entries.append(StepEntry(t.seq.id, t.token_ids, [len(t.token_ids) - 1] if t.completes else []))
            if t.completes:
                rows.append(self._row(t.seq))
        try:
            logits = self.engine.step(entries)
            tokens = self.sampler.select(logits, rows)
        except Exception as e:                    # the requests of this batch end with an error event
            for t in list(plan.decode) + list(plan.prefill):
                self.scheduler._fail(t.seq, f"{type(e).__name__}: {e}")
            raise
        self.steps += 1
        self.tokens_run += plan.num_tokens
        k = 0
        for t in plan.decode:
            self.scheduler.on_decode_done(t, tokens[k])
            k += 1
        for t in plan.prefill:
            if t.completes:
                self.scheduler.on_prefill_done(t, tokens[k])
                k += 1
            else:
                self.scheduler.on_prefill_done(t, None)
        return plan

    # ---- one step ahead ------------------------------------------------------------------
    def _all_can_wait(self) -> bool:
        if getattr(self.sampler, "history_on_device", False):
            return True                           # the sampler finds a request's newest token on the device
        needs = self.sampler.needs_history
        return not any(needs(s.options.sampling) for s in self.scheduler.running) and \
            not any(needs(s.options.sampling) for s in self.scheduler.waiting)

    def _deliver(self) -> None:
        """The tokens of the step in flight, if any, go to their requests."""
        flight, self._inflight = self._inflight, None
        if flight is None:
            return
        plan, handle = flight[0], flight[3]
        tokens = self._download.wait(handle)
        k = 0
        for t in plan.decode:
            self.scheduler.on_decode_done(t, tokens[k])
            k += 1
        for t in plan.prefill:
            if t.completes:
                self.scheduler.on_prefill_done(t, tokens[k])
                k += 1

    def _step_ahead(self) -> SchedulerOutput:
        plan = self.scheduler.step(self.engine.cache)
        if plan.is_empty():
            self._deliver()
            return plan
        before = self._inflight
        row_before = before[2] if before is not None else {}
        entries: List[StepEntry] = []
        rows: List[RowRequest] = []
        index: List[int] = []
        row_of = {}
        for t in plan.decode:
            s = t.seq
            if s.pending:                         # its last token is where the step in flight leaves it
                entries.append(StepEntry(s.id, [0], [0]))
                index.append(row_before[s.id])
            else:
                entries.append(StepEntry(s.id, [s.generated_ids[-1]], [0]))
                index.append(-1)
            row_of[s.id] = len(rows)
            rows.append(self._row(s, index[-1]))
        for t in plan.prefill:
            entries.append(StepEntry(t.seq.id, t.token_ids, [len(t.token_ids) - 1] if t.completes else []))
            index.append(-1)
            if t.completes:
                row_of[t.seq.id] = len(rows)
                rows.append(self._row(t.seq))
        try:
            feed = (before[1], index) if before is not None and any(j >= 0 for j in index) else None
            logits = self.engine.step(entries, device_tokens=feed, borrow_logits=True)
            if any(r.pending_row >= 0 for r in rows):
                chosen = self.sampler.select_on_device(logits, rows, previous=before[1])
            else:
                chosen = self.sampler.select_on_device(logits, rows)
        except Exception as e:                    # the requests of this batch end with an error event
            for t in list(plan.decode) + list(plan.prefill):
                self.scheduler._fail(t.seq, f"{type(e).__name__}: {e}")
            self._deliver()
            raise
        self.steps += 1
        self.tokens_run += plan.num_tokens
        self.scheduler.on_launched(plan)
        if self._download is None:
            device = getattr(getattr(self.engine, "rt", None), "device", None)
            if device is not None and device.type == "cuda":
                from ..kernels.staging import TokenDownload
                self._download = TokenDownload(device)
            else:
                self._download = _TokensAtHand()
        handle = self._download.start(chosen)
        self._deliver()                           # the step before: its tokens while this one runs
        self._inflight = (plan, chosen, row_of, handle)
        return plan

    @staticmethod
    def _row(s: SequenceState, pending_row: int = -1) -> RowRequest:
        """``pending_row`` >= 0: the request's newest token is that entry of the tokens which the step in flight
        leaves on the device; the host's list then ends one token earlier."""
        sp = s.options.sampling
        if sp is None:
            return RowRequest(None)
        hist: Sequence[int] = ()
        looks_back = abs(sp.repetition_penalty - 1.0) > 1.1920929e-07 and sp.repetition_penalty_window > 0
        if looks_back:
            # the last tokens of prompt and generation that the penalty looks at, not the whole sequence
            n = sp.repetition_penalty_window - (1 if pending_row >= 0 else 0)
            hist = s.generated_ids[-n:] if n > 0 else []
            if len(hist) < n:
                hist = s.prompt_ids[len(s.prompt_ids) - min(n - len(hist), len(s.prompt_ids)):] + hist
        return RowRequest(sp, len(s.generated_ids) + s.pending, hist, pending_row if looks_back else -1)

    def run(self, until: Optional[Callable[[], bool]] = None) -> None:
        """Step until nothing waits or runs (or until ``until()`` is true)."""
        while not self.scheduler.is_idle():
            if until is not None and until():
                return
            self.step()
        if until is None or self.scheduler.is_idle():
            self._deliver()
        self.scheduler.reap(self.engine.cache)

    # ---- whole generations ---------------------------------------------------------------
    def generate(self, prompt: Prompt, options: Optional[GenerateOptions] = None) -> Union[str, List[int]]:
        """Blocks until done.  A list of token ids gives a list of new token ids (engine.rs:132-145);
        a string is encoded with the tokenizer, the end-of-sequence id is filled in from the model's
        configuration when the options name none, and the new text comes back (runtime.rs:81-97)."""
        ids, options, is_text = self._prepare(prompt, options)
        out = self.generate_batch([ids], options)[0]
        return self.tokenizer.decode(out) if is_text else out

    def generate_batch(self, prompts: Sequence[Sequence[int]],
                       options: Union[None, GenerateOptions, Sequence[GenerateOptions]] = None) -> List[List[int]]:
        """Several requests at once through continuous batching; new token ids of each, in order."""
        if options is None or isinstance(options, GenerateOptions):
            options = [options or GenerateOptions()] * len(prompts)
        if len(options) != len(prompts):
            raise ValueError("one GenerateOptions per prompt, or one for all")
        if any(not o.use_kv_cache for o in options):
            return [self._generate_without_cache(p, o) for p, o in zip(prompts, options)]
        seqs = [self.submit(p, o) for p, o in zip(prompts, options)]
        self.run(until=lambda: all(s.phase == SequencePhase.FINISHED for s in seqs))
        self.scheduler.reap(self.engine.cache)
        for s in seqs:
            if s.error is not None:
                raise GenerationError(s.error)
        return [list(s.generated_ids) for s in seqs]

    def generate_stream(self, prompt: Prompt, options: Optional[GenerateOptions] = None) -> Iterator[Union[int, str]]:
        """Yields each new token (its text for a string prompt) as soon as it is chosen (engine.rs:148-170)."""
        ids, options, is_text = self._prepare(prompt, options)
        fresh: List[int] = []
        seq = self.submit(ids, options, lambda ev: (fresh.append(ev.token) if ev.kind == "token" else None, True)[1])
        try:
            while seq.phase != SequencePhase.FINISHED or fresh:
                if not fresh:
                    self.step()
                while fresh:
                    t = fresh.pop(0)
                    yield self.tokenizer.decode([t]) if is_text else t
        finally:
            self.scheduler.cancel(seq)            # a consumer that stops early cancels the request
            self.scheduler.reap(self.engine.cache)
        if seq.error is not None:
            raise GenerationError(seq.error)

    def _prepare(self, prompt: Prompt, options: Optional[GenerateOptions]):
        options = options or GenerateOptions()
        if options.eos_token_id is None:
            # the model's end-of-sequence token stands in for every request that names none
            # (infernum-runtime/src/runtime.rs:127-134); ``submit`` takes the options as they are
            eos = getattr(getattr(self.engine, "spec", None), "eos_token_id", None)
            options = GenerateOptions(options.max_new_tokens, eos, options.sampling, options.use_kv_cache)
        if isinstance(prompt, str):
            if self.tokenizer is None:
                raise GenerationError("a text prompt needs a tokenizer (tokenizer.json in the model folder); "
                                      "pass token ids instead")
            return self.tokenizer.encode(prompt, add_bos=True), options, True
        return [int(t) for t in prompt], options, False

    def _generate_without_cache(self, prompt: Sequence[int], options: GenerateOptions) -> List[int]:
        """Every new token from the whole sequence, computed afresh (GenerateOptions.use_kv_cache = false)."""
        toks, out = [int(t) for t in prompt], []
        probe = SequenceState("nocache", toks, options)
        limit = getattr(getattr(self.engine, "rt", None), "max_tokens_per_step", None) or (1 << 30)
        self._recomputed += 1
        name = ("recomputed", self._recomputed)         # a name that no request of the scheduler has
        for _ in range(options.max_new_tokens):
            whole = toks + out
            try:
                for p in range(0, len(whole), limit):       # longer than a step takes: in portions
                    part = whole[p:p + limit]
                    logits = self.engine.step([StepEntry(name, part, [len(part) - 1] if p + limit >= len(whole) else [])])
            finally:
                self.engine.end(name)
            probe.generated_ids = out
            tok = self.sampler.select(logits, [self._row(probe)])[0]
            if options.eos_token_id is not None and tok == options.eos_token_id:
                break
            out = out + [tok]
        return out


class TextTokenizer:
    """tokenizer.json of a model folder through the ``tokenizers`` library."""

    def __init__(self, path: str, bos_token_id: Optional[int] = None):
        from tokenizers import Tokenizer
        self._tok = Tokenizer.from_file(path)
        self.bos_token_id = bos_token_id

    def encode(self, text: str, add_bos: bool = True) -> List[int]:
        ids = list(self._tok.encode(text, add_special_tokens=False).ids)
        if add_bos and self.bos_token_id is not None and (not ids or ids[0] != self.bos_token_id):
            ids = [self.bos_token_id] + ids
        return ids

    def decode(self, ids: Sequence[int]) -> str:
        return self._tok.decode(list(ids), skip_special_tokens=True)


def load_tokenizer(model_dir: str) -> Optional[TextTokenizer]:
    path = os.path.join(model_dir, "tokenizer.json")
    if not os.path.isfile(path):
        return None
    from ..config.registry import load_config
    return TextTokenizer(path, getattr(load_config(model_dir), "bos_token_id", None))

"""The scheduler's decisions once more, plainly: the rules of ``Scheduler.step`` written out in Python over the
cache manager's public counts.  ``tests/test_scheduler_plain.py`` runs it beside the product's scheduler (whose
decisions are taken natively) on the same requests and compares every step."""
from typing import List

from infernum_amd.cache import CacheManager
from infernum_amd.engine.scheduler import (DecodeTask, PrefillTask, Scheduler, SchedulerOutput, SequencePhase,
                                           SequenceState)


class PlainScheduler(Scheduler):
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

        def cut(n: int, remaining: int) -> int:
            """A portion that does not reach its prompt's end stops where the step's tokens are a multiple of
            ``step_token_multiple``, if that leaves it at least half of what it could take."""
            m = cfg.step_token_multiple
            if m <= 1 or n >= remaining:
                return n
            used = cfg.max_tokens_per_step - budget
            whole = (used + n) // m * m
            return whole - used if (whole - used) * 2 >= n else n

        # requests that are done but for a token still on its way: they hold their pages, do nothing, are never
        # set back; who cannot move because of them waits
        leaving = [s for s in self.running if self._awaits_last_token(s)]
        movable = lambda: [s for s in self.running if s not in leaving]        # noqa: E731

        # 2. one token for every decoding request
        i = 0
        while i < len(self.running):
            seq = self.running[i]
            if seq.phase != SequencePhase.DECODE or seq in leaving:
                i += 1
                continue
            need = cache.pages_needed(seq.id, 1)
            if fits(need):
                take(need)
                budget -= 1
                out.decode.append(DecodeTask(seq))
                i += 1
                continue
            if leaving:
                i += 1
                continue
            victim = movable()[-1]
            if victim is seq and len(movable()) == 1:
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
            if n > 0:
                n = cut(n, seq.num_tokens - cached)
            if n <= 0:
                if out.is_empty() and not leaving:
                    # nobody can move: the last admitted request makes room
                    victim = movable()[-1]
                    if victim is seq and len(movable()) == 1:
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
            n = cut(min(seq.num_tokens, cfg.max_prefill_tokens, budget), seq.num_tokens)
            need = cache.pages_needed(seq.id, n)
            # keep one page in hand for every running request, so that a newcomer is not set back at once
            spare = [len(self.running)] * len(need) if self.running else [0] * len(need)
            if not fits([a + b for a, b in zip(need, spare)]):
                if not self.running and out.is_empty():
                    # alone and still too large for one portion: shrink the portion to the pool
                    n = min(n, cache.tokens_that_fit(None, promised))
                    if n > 0:
                        n = cut(n, seq.num_tokens)
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

"""The scheduler: admits requests, cuts prompts into portions under a token budget,
decodes, finishes and frees.

The reference's `Pipeline::apply` has none of this: a fixed list of prompts is
prefilled whole in one step, every request then decodes in lockstep, finished
requests are fed eos until request 0 reaches `max_new_tokens`, and all pages go back
at the very end (tiny_llm/pipeline/pipeline.cpp:118-130, 181-231).  Kept from it: the
position rule `pos = prompt_len + generated - 1` for a decoded token (:224-225), eos
ends a request and is part of its output (:216-223), `max_new_tokens` bounds it.

Decisions (all host-side, testable without a GPU):
* A request's tokens are prompt + output; `num_computed` of them are in the cache.
  Each step it is fed the next portion; when the portion reaches the end, the last
  logits are wanted and a token is sampled.  Decoding is the portion of one.
* Order within a step: running requests first, those that decode before those still
  in their prompt, each group in order of admission; then waiting requests are
  admitted in arrival order while a request slot, blocks for their first portion and
  token budget are left.
* Budget: at most `max_num_batched_tokens` tokens per step; a prompt portion is
  `min(remaining, budget left, blocks that fit)`.
* A waiting request is admitted only when, in every cache group, the blocks it will
  hold at most are free: all its tokens in a group that keeps every position, its
  window and one portion in a group that keeps a window (its first portion may still
  be shorter: the token budget).
* When pages run out for a running request, the request admitted last among those
  not yet scheduled in the step (possibly the request itself) is preempted: its
  blocks and slot are given back at once and it returns to the FRONT of the waiting
  queue with nothing computed; prompt and output so far are recomputed when it is
  admitted again.  No request is admitted in a step that preempted.  A request that
  cannot go on even alone, with every other block free, is finished with reason
  "capacity": the engine never deadlocks.
"""
from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field
from typing import Deque, Dict, Hashable, List, Optional, Sequence

from ..cache import CacheManager
from ..sampling.params import SamplingParams

WAITING, RUNNING, FINISHED = "waiting", "running", "finished"


@dataclass(eq=False)          # a request is itself: membership tests compare identities, not token lists
class Request:
    req_id: Hashable
    prompt: List[int]
    params: SamplingParams
    seed: int = 0
    output: List[int] = field(default_factory=list)
    num_computed: int = 0
    status: str = WAITING
    finish_reason: Optional[str] = None
    preemptions: int = 0

    @property
    def tokens(self) -> List[int]:
        return self.prompt + self.output

    @property
    def num_tokens(self) -> int:
        return len(self.prompt) + len(self.output)

    @property
    def pending(self) -> int:
        return self.num_tokens - self.num_computed

    def token_slice(self, start: int, count: int) -> List[int]:
        """tokens[start:start + count] without building the whole list."""
        n = len(self.prompt)
        if start >= n:
            return self.output[start - n:start - n + count]
        if start + count <= n:
            return self.prompt[start:start + count]
        return self.prompt[start:] + self.output[:start + count - n]


@dataclass
class Scheduled:
    request: Request
    start: int          # first token position fed this step
    count: int          # number of tokens fed
    samples: bool       # the portion reaches the end: its last logits are wanted


@dataclass
class StepPlan:
    entries: List[Scheduled]
    preempted: List[Request]
    finished: List[Request]      # requests finished by the scheduler itself (reason "capacity")

    @property
    def num_tokens(self) -> int:
        return sum(e.count for e in self.entries)


class Scheduler:
    FINISHED_KEPT = 4096

    def __init__(self, cache: CacheManager, max_num_seqs: int, max_num_batched_tokens: int, max_model_len: int,
                 eos_token_id=None):
        """eos_token_id: one id, several, or None (nothing ends a request but its length)."""
        self.cache = cache
        self.max_num_seqs = int(max_num_seqs)
        self.budget = int(max_num_batched_tokens)
        self.max_model_len = int(max_model_len)
        self.eos_token_id = eos_token_id
        self.waiting: Deque[Request] = deque()
        self.running: List[Request] = []       # in order of admission
        # the requests that finished last (a bounded record: a serving process finishes without end)
        self.finished: Deque[Request] = deque(maxlen=self.FINISHED_KEPT)

    @property
    def eos_token_id(self):
        return self._eos

    @eos_token_id.setter
    def eos_token_id(self, value) -> None:
        self._eos = value
        if value is None:
            self.eos_token_ids = frozenset()
        elif isinstance(value, (list, tuple, set, frozenset)):
            self.eos_token_ids = frozenset(int(v) for v in value)
        else:
            self.eos_token_ids = frozenset([int(value)])

    # ---------------------------------------------------------------- requests
    def add(self, req: Request) -> None:
        if not req.prompt:
            raise ValueError("a request needs at least one prompt token")
        if len(req.prompt) > self.max_model_len:
            raise ValueError(f"prompt of {len(req.prompt)} tokens exceeds max_model_len {self.max_model_len}")
        alone = self.cache.blocks_held_at_most(len(req.prompt), self.budget)
        if any(n > have for n, have in zip(alone, self.cache.group_blocks)):
            raise ValueError(f"prompt of {len(req.prompt)} tokens cannot fit the cache: it holds up to {alone} "
                             f"blocks of {self.cache.block_size}, the pools have {self.cache.group_blocks}")
        req.status = WAITING
        self.waiting.append(req)

    def has_work(self) -> bool:
        return bool(self.waiting or self.running)

    def abort(self, req_id) -> None:
        for r in list(self.running):
            if r.req_id == req_id:
                self._finish(r, "abort")
        for r in list(self.waiting):
            if r.req_id == req_id:
                self.waiting.remove(r)
                r.status, r.finish_reason = FINISHED, "abort"
                self.finished.append(r)

    # ---------------------------------------------------------------- planning
    def _needs(self, req: Request, count: int) -> List[int]:
        return self.cache.blocks_needed(req.req_id, req.num_computed + count)

    def _fits(self, need: Sequence[int], taken: Sequence[int]) -> bool:
        free = self.cache.free_blocks()
        return all(n + t <= f for n, t, f in zip(need, taken, free))

    def _largest_fit(self, req: Request, want: int, taken: Sequence[int]) -> int:
        """Largest portion <= want whose blocks are free now (0 if not even one token)."""
        free = self.cache.free_blocks()
        bs = self.cache.block_size
        have = [len(self.cache.block_table(req.req_id, g)) if self.cache.has(req.req_id) else 0
                for g in range(len(free))]
        room = min((h + f - t) * bs for h, f, t in zip(have, free, taken)) if free else 1 << 60
        return max(0, min(want, room - req.num_computed))

    def _preempt(self, victim: Request) -> None:
        if self.cache.has(victim.req_id):
            self.cache.free_request(victim.req_id)
        self.running.remove(victim)
        victim.num_computed = 0
        victim.status = WAITING
        victim.preemptions += 1
        self.waiting.appendleft(victim)

    def _finish(self, req: Request, reason: str) -> None:
        if self.cache.has(req.req_id):
            self.cache.free_request(req.req_id)
        if req in self.running:
            self.running.remove(req)
        req.status, req.finish_reason = FINISHED, reason
        self.finished.append(req)

    def schedule(self) -> StepPlan:
        entries: List[Scheduled] = []
        preempted: List[Request] = []
        finished: List[Request] = []
        taken = [0] * len(self.cache.groups)
        budget = self.budget

        order = [r for r in self.running if r.pending == 1] + [r for r in self.running if r.pending > 1]
        scheduled_ids = set()
        for req in order:
            if req.status != RUNNING or budget <= 0:      # preempted meanwhile / no budget left
                continue
            want = min(req.pending, budget)
            if want == 1 and self.cache.has_room(req.req_id, req.num_computed + 1):
                # the usual decoded token: its block is there already, nothing to weigh
                entries.append(Scheduled(req, req.num_computed, 1, req.num_computed + 1 == req.num_tokens))
                scheduled_ids.add(req.req_id)
                budget -= 1
                continue
            while True:
                count = self._largest_fit(req, want, taken)
                if count >= 1 and (count == want or req.pending > 1):
                    break
                # Not even the next token fits.  The request admitted last among those not yet
                # scheduled in this step gives its blocks back; that may be this request itself.
                victim = next(r for r in reversed(self.running) if r.req_id not in scheduled_ids)
                if victim is req:
                    count = 0
                    if len(self.running) == 1 and not entries:
                        self._finish(req, "capacity")      # alone, every other block free: it can never go on
                        finished.append(req)
                    else:
                        self._preempt(req)
                        preempted.append(req)
                    break
                self._preempt(victim)
                preempted.append(victim)
            if count == 0:
                continue
            need = self._needs(req, count)
            taken = [t + n for t, n in zip(taken, need)]
            entries.append(Scheduled(req, req.num_computed, count, req.num_computed + count == req.num_tokens))
            scheduled_ids.add(req.req_id)
            budget -= count

        # Admission, in arrival order, while a slot, the blocks the request will hold at most (in a
        # full group: for ALL its tokens) and some budget are left; none in a step that preempted
        # (the freed blocks are for those that run).
        slots_left = min(self.cache.free_slots, self.max_num_seqs - len(self.running))
        while self.waiting and budget > 0 and slots_left > 0 and not preempted:
            req = self.waiting[0]
            need_all = self.cache.blocks_held_at_most(req.num_tokens, self.budget)
            if not self._fits(need_all, taken):
                if any(n > have for n, have in zip(need_all, self.cache.group_blocks)):
                    self.waiting.popleft()                 # more than the whole pool: it can never run
                    req.status, req.finish_reason = FINISHED, "capacity"
                    self.finished.append(req)
                    finished.append(req)
                    continue
                break
            count = min(req.pending, budget)
            self.waiting.popleft()
            req.status = RUNNING
            self.running.append(req)
            need = self._needs(req, count)
            taken = [t + n for t, n in zip(taken, need)]
            entries.append(Scheduled(req, req.num_computed, count, req.num_computed + count == req.num_tokens))
            scheduled_ids.add(req.req_id)
            budget -= count
            slots_left -= 1
        return StepPlan(entries, preempted, finished)

    def burst_length(self, plan: StepPlan, most: int) -> int:
        """How many decode steps the plan's requests can run back to back without a decision in
        between: every entry decodes, every running request is in the plan, nobody waits for
        admission, and the run ends where the
        first request reaches its `max_new_tokens` or the model's length, where the requests would
        need cache blocks that are not free, or after `most` steps.  (A request that draws an end-of-
        sequence token inside the run is finished there when the run is over; what it was given
        after that token is dropped.)"""
        if most < 2 or self.waiting or plan.preempted or not plan.entries:
            return 1
        if len(plan.entries) != len(self.running):
            return 1            # a running request the plan left out (no budget) would sit idle for the whole run
        k = most
        for e in plan.entries:
            req = e.request
            if e.count != 1 or not e.samples:
                return 1
            k = min(k, req.params.max_new_tokens - len(req.output), self.max_model_len - req.num_tokens)
        if k < 2:
            return 1
        # the longest run whose blocks are free now, in every group (all of them are taken up front)
        free = self.cache.free_blocks()
        while k >= 2:
            need = [0] * len(free)
            for e in plan.entries:
                for g, n in enumerate(self.cache.blocks_needed(e.request.req_id, e.request.num_computed + k)):
                    need[g] += n
            if all(n <= f for n, f in zip(need, free)):
                return k
            k -= 1
        return 1

    def update_burst(self, plan: StepPlan, tokens_by_step: Sequence[Sequence[int]]) -> List[Request]:
        """After a run of decode steps: what `update` would do with each step's tokens in turn, worked
        out per request (a request that finishes at one step takes no part in the later ones; what
        it was given after that step is dropped).  Returns the finished requests in the order in
        which `update` would have finished them."""
        steps = len(tokens_by_step)
        eos = self.eos_token_ids
        ended = []
        for i, e in enumerate(plan.entries):
            req = e.request
            toks = [int(step[i]) for step in tokens_by_step]
            # the first step at which `update` would finish the request (1-based), if any
            by_length = min(req.params.max_new_tokens - len(req.output), self.max_model_len - req.num_tokens)
            by_length = max(by_length, 1)
            by_eos = steps + 1
            if eos and not req.params.ignore_eos:
                for k, t in enumerate(toks):
                    if t in eos:
                        by_eos = k + 1
                        break
            take = min(steps, by_length, by_eos)
            req.output.extend(toks[:take])
            req.num_computed = e.start + take
            reason = "stop" if by_eos == take else ("length" if by_length == take else None)
            if reason:
                ended.append((take, i, req, reason))
        done: List[Request] = []
        for _, _, req, reason in sorted(ended, key=lambda x: (x[0], x[1])):
            self._finish(req, reason)
            done.append(req)
        return done

    # ------------------------------------------------------------------ results
    def update(self, plan: StepPlan, sampled: Dict[Hashable, int]) -> List[Request]:
        """After the step ran: advances every scheduled request, appends sampled tokens,
        finishes and frees.  Returns the requests that finished now."""
        done: List[Request] = []
        for e in plan.entries:
            req = e.request
            req.num_computed = e.start + e.count
            if not e.samples:
                continue
            tok = int(sampled[req.req_id])
            req.output.append(tok)
            reason = None
            if tok in self.eos_token_ids and not req.params.ignore_eos:
                reason = "stop"
            elif len(req.output) >= req.params.max_new_tokens:
                reason = "length"
            elif req.num_tokens >= self.max_model_len:
                reason = "length"
            if reason:
                self._finish(req, reason)
                done.append(req)
        return done

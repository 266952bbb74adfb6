"""Which requests run in the next step, and with how many tokens each.

The reference admits a request when a row is free, reserves its worst case of
pages, prefills the whole prompt alone, and then decodes all rows together
(model/inference_paged.py:150-179, 231-237); pages cannot run out by
construction (:9-13). Here pages are taken step by step, prompts are cut into
portions under a token budget and run beside the decoding rows, and the case
that pages run out is decided as follows:

* A request's next tokens are whatever its cache does not hold yet of prompt +
  output: a portion of the prompt, one decoded token, or, after a preemption,
  both again. A portion that reaches the last of them asks for logits.
* Running requests are served oldest first. One that cannot get its pages takes
  them from the youngest running requests: those are *preempted* (row closed,
  pages freed, put back at the head of the queue with their output kept; their
  cache is recomputed later as a prompt portion). If none is younger, a prompt
  portion is shortened to what fits, and otherwise the request waits; the oldest
  request always fits, because ``submit`` refuses what the whole pool cannot hold.
* New requests are admitted in arrival order while a row and budget are free and the
  pool has pages for all tokens the request has so far plus one, and only if no
  running request had to wait or was preempted in this step.
"""

from __future__ import annotations

import time
from collections import deque
from dataclasses import dataclass
from typing import List

from ..cache import CacheManager
from .request import QueueFull, Request, TooLong


@dataclass
class Planned:
    request: Request
    tokens: List[int]
    wants_logits: bool


class Scheduler:
    def __init__(self, cache: CacheManager, max_batch: int, max_len: int, token_budget: int,
                 max_queue: int):
        if token_budget < 1 or max_batch < 1:
            raise ValueError("token_budget and max_batch must be positive")
        self.cache = cache
        self.max_batch = min(max_batch, cache.max_rows)
        self.max_len = min(max_len, cache.max_len)
        self.token_budget, self.max_queue = token_budget, max_queue
        self.pending = deque()
        self.running: List[Request] = []          # in order of admission, oldest first
        self.n_preemptions = 0

    # -- queue -----------------------------------------------------------------------------
    def submit(self, req: Request) -> None:
        if len(self.pending) >= self.max_queue:
            raise QueueFull(f"{len(self.pending)} requests already waiting")
        if not req.ids:
            raise ValueError("a request needs at least one prompt token")
        total = len(req.ids) + req.max_new_tokens
        limit = min(self.max_len, self.cache.pool_tokens)
        if total > limit:
            raise TooLong(f"prompt is {len(req.ids)} tokens; with {req.max_new_tokens} new it exceeds "
                          f"the {limit} tokens one request can hold")
        self.pending.append(req)

    @property
    def idle(self) -> bool:
        return not self.pending and not self.running

    # -- one step's plan ---------------------------------------------------------------------
    def _cached(self, req: Request) -> int:
        return self.cache.length(req.row)

    @staticmethod
    def _todo(req: Request, cached: int) -> List[int]:
        """The tokens of prompt + output that the cache does not hold yet."""
        n_prompt = len(req.ids)
        if cached >= n_prompt:
            return req.output[cached - n_prompt:]
        return req.ids[cached:] + req.output

    def _fits(self, need, free) -> bool:
        return all(n <= f for n, f in zip(need, free))

    def _preempt(self, victim: Request) -> None:
        self.cache.close_row(victim.row)
        victim.row = -1
        victim.preemptions += 1
        self.n_preemptions += 1
        self.running.remove(victim)
        self.pending.appendleft(victim)

    def _admit(self, req: Request, row: int) -> None:
        """Give ``req`` the row and put its sampling state into the row's fixed-size state. A
        request that comes back after a preemption continues its random stream where it
        stopped: one draw per token it has produced."""
        req.row = row
        if not req.admitted:
            req.admitted = time.perf_counter()
        scalars = self.cache.scalars
        scalars.temperature[row] = req.sampling.temperature
        scalars.seed[row] = req.sampling.seed & 0x7FFFFFFFFFFFFFFF
        scalars.draws[row] = len(req.output)
        self.running.append(req)

    def _longest_fit(self, row: int, cached: int, n: int, free) -> int:
        """The most of ``n`` next tokens of ``row`` whose pages fit into ``free``."""
        lo, hi = 0, n
        while lo < hi:                        # need is monotone in the number of tokens
            mid = (lo + hi + 1) // 2
            if self._fits(self.cache.pages_needed(row, cached + mid), free):
                lo = mid
            else:
                hi = mid - 1
        return lo

    def plan(self) -> List[Planned]:
        """Retire what is finished, then choose the next step's entries. Preempts and
        admits as a side effect. An empty plan means there is nothing to run."""
        self.retire_finished()
        if any(r.cancelled for r in self.pending):
            for r in self.pending:
                if r.cancelled:
                    r.event.set()
            self.pending = deque(r for r in self.pending if not r.cancelled)
        cache = self.cache
        plan: List[Planned] = []
        budget = self.token_budget
        free = cache.free_pages()
        someone_waits = False
        i = 0
        while i < len(self.running):
            req = self.running[i]
            i += 1
            if budget == 0:
                someone_waits = True
                break
            cached = self._cached(req)
            todo = self._todo(req, cached)
            n = min(len(todo), budget)
            need = cache.pages_needed(req.row, cached + n)
            while not self._fits(need, free) and self.running[-1] is not req:
                self._preempt(self.running[-1])          # youngest first; never one already planned
                someone_waits = True                     # and nobody is admitted in this step
                free = cache.free_pages()
                for p in plan:                           # pages promised to earlier entries
                    taken = cache.pages_needed(p.request.row, self._cached(p.request) + len(p.tokens))
                    free = [f - max(t, 0) for f, t in zip(free, taken)]
            if not self._fits(need, free):
                n = self._longest_fit(req.row, cached, n, free) if len(todo) > 1 else 0
                if n == 0:
                    if not plan and req is self.running[0]:
                        raise RuntimeError("the oldest request cannot get a page: the pool is smaller "
                                           "than one request, which submit() should have refused")
                    someone_waits = True
                    continue
                need = cache.pages_needed(req.row, cached + n)
            plan.append(Planned(req, todo[:n], n == len(todo)))
            free = [f - max(t, 0) for f, t in zip(free, need)]
            budget -= n
        # admission, in arrival order
        while (self.pending and not someone_waits and budget > 0
               and len(self.running) < self.max_batch and cache.n_free_rows > 0):
            req = self.pending[0]
            if req.cancelled:
                self.pending.popleft()
                req.event.set()
                continue
            todo = req.tokens()
            row = cache.open_row()
            n = min(len(todo), budget)
            # Pages for everything the request has so far, and its next token, must be free
            # (else it would soon take pages from, or be preempted by, the running ones).
            if not self._fits(cache.pages_needed(row, len(todo) + 1), free):
                if self.running:
                    cache.close_row(row)
                    break
                n = self._longest_fit(row, 0, n, free)      # alone: the pool is as free as it gets
            if n == 0:
                cache.close_row(row)
                break
            self.pending.popleft()
            self._admit(req, row)
            need = cache.pages_needed(row, n)
            plan.append(Planned(req, todo[:n], n == len(todo)))
            free = [f - max(t, 0) for f, t in zip(free, need)]
            budget -= n
        return plan

    def repeats(self, plan: List[Planned]) -> bool:
        """Whether the step after ``plan`` is known before ``plan``'s tokens are: every
        running request gets a token from ``plan`` and none reaches its limit with it, nobody
        is cancelled, nobody who waits could be given a row, and the pages for one more token
        each are free, so that the next step is one token for each of the same requests
        whatever the tokens turn out to be (a stop token aside: its request's place in that
        next step is then wasted, and whoever waits for its row gets it a step later).
        Changes nothing."""
        if len(plan) != len(self.running):
            return False
        if self.pending and len(self.running) < self.max_batch and self.cache.n_free_rows > 0:
            return False
        free = self.cache.free_pages()
        for p, req in zip(plan, self.running):
            if (p.request is not req or not p.wants_logits or req.cancelled or req.done
                    or len(req.output) + 1 >= req.max_new_tokens):
                return False
            need = self.cache.pages_needed(req.row, self._cached(req) + 1)
            if not self._fits(need, free):
                return False
            free = [f - max(t, 0) for f, t in zip(free, need)]
        return True

    # -- finishing ---------------------------------------------------------------------------
    def retire_finished(self) -> List[Request]:
        """Close the rows of requests that are done or cancelled; their pages are free
        for the step planned next."""
        gone = [r for r in self.running if r.done or r.cancelled]
        for req in gone:
            self.cache.close_row(req.row)
            req.row = -1
            self.running.remove(req)
            req.event.set()
        return gone

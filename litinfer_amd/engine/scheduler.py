"""The scheduler above the step function: it admits requests, cuts prompts into
portions under a token budget, decodes, finishes and frees.

Every step it plans one batch:
 1. one token for every running request that is decoding;
 2. the rest of the token budget to running requests still in their prompt,
    oldest first, each at most `chunk_size` tokens and no more than the free
    pages allow; a portion that does not reach the prompt's end asks for no
    logits;
 3. requests from the waiting queue, first come first served, while budget and
    a state slot remain and the free pages cover all of the request's prompt.
When the pages do not even cover the decoding requests, the most recently
admitted running request is PREEMPTED: all it holds is given back, it goes to
the head of the waiting queue, and when it is admitted again its prompt plus
what it had generated is computed anew (its random stream goes on where it
was, so its tokens are the same as without preemption).  A request that could
never fit the pool alone is refused when it is submitted.

The reference admits every request into the very next step whole, without a
budget or a look at the free pages, and when its pool is full the step throws
and the caller spins (src/llaisys/models/qwen2.cpp:789-800, 832-845, 925-944;
serving/engine_runtime.py:42-62).  Its finishing rules are kept: an end token
is dropped and ends the request, the token that reaches max_new_tokens is kept
(:1058-1073).

With `lookahead` the scheduler does not wait for a step's sampled tokens before
it plans and starts the next step: the sampler leaves them in the engine's
feedback buffer on the device, the next step's entries take them from there,
and the host reads them one step later, while the device is already at work.
What can only be known from a token's value (an end token) is found out one
step late: the request has then run one token too far, which is dropped.  What
is counted (max_new_tokens, the model's length) is foreseen, and such a request
is not run again until its last token has arrived.  The tokens are the same
with and without it.
"""
from __future__ import annotations

import itertools
from collections import deque
from dataclasses import dataclass, field
from typing import Deque, Dict, Hashable, List, Optional, Sequence, Tuple

import numpy as np

from ..cache import CacheFull
from ..sampling import Sampler, SamplingParams
from .batch import StepEntry

WAITING, RUNNING, FINISHED = "waiting", "running", "finished"


@dataclass
class Request:
    rid: Hashable
    prompt: List[int]
    max_new_tokens: int
    params: Optional[SamplingParams]
    first_token_greedy: bool = False
    state: str = WAITING
    generated: List[int] = field(default_factory=list)
    computed: int = 0                # tokens of prompt + generated that are in the cache
    samples_drawn: int = 0           # position in the request's random stream
    finish_reason: Optional[str] = None
    preemptions: int = 0
    arrival: int = 0
    # lookahead: the request's newest token has been sampled but is not known here yet; it lies
    # at this place of the engine's feedback buffer
    pending_take: Optional[int] = None
    # the state slot and the options that the sampler's table on the device holds for this request
    # (None: not written yet, or the request has given its slot back)
    bound: Optional[Tuple[int, SamplingParams]] = None

    @property
    def num_generated(self) -> int:
        return len(self.generated) + (self.pending_take is not None)

    @property
    def tokens(self) -> List[int]:
        """Prompt and generated tokens; a pending token stands as 0 (its entry takes the id from
        the feedback buffer)."""
        return self.prompt + self.generated + ([0] if self.pending_take is not None else [])

    @property
    def remaining(self) -> int:
        return len(self.prompt) + self.num_generated - self.computed

    def slice_tokens(self, start: int, n: int) -> List[int]:
        """tokens[start:start + n] without putting the whole list together."""
        lp = len(self.prompt)
        if start + n <= lp:
            return self.prompt[start:start + n]
        out = self.prompt[start:] if start < lp else []
        out = out + self.generated[max(start - lp, 0):start + n - lp]
        if len(out) < n:
            out.append(0)                              # the pending token's place
        return out


class _Ready:
    """Tokens that a sampler without an asynchronous call has already brought."""
    def __init__(self, tokens):
        self._tokens = list(tokens)

    def result(self):
        return self._tokens


@dataclass
class Planned:
    request: Request
    start: int
    n: int
    wants_logits: bool


class Scheduler:
    def __init__(self, engine, *, max_batch_tokens: int = 2048, chunk_size: int = 512,
                 max_running: Optional[int] = None, eos_token_ids: Optional[Sequence[int]] = None,
                 sampler=None, lookahead: bool = False, row_tile: Optional[int] = None):
        """row_tile: rows that the kernels of a step take at a time (the products' tiles).  A step
        whose tokens number a few more than a multiple of it (up to half a tile) pays for a whole
        tile more: then the last portion of a prompt in the plan that is not the prompt's end gives
        those tokens up to the next step.  1: as planned.  None: what the engine's model says
        (`Engine.row_tile`, the largest `BatchNeeds.row_tile` of its parts)."""
        if row_tile is None:
            row_tile = int(getattr(engine, "row_tile", 1) or 1)
        if max_batch_tokens <= 0 or chunk_size <= 0 or row_tile <= 0:
            raise ValueError("scheduler: max_batch_tokens, chunk_size and row_tile must be positive")
        self.engine = engine
        self.cache = engine.cache
        self.max_batch_tokens = int(max_batch_tokens)
        self.chunk_size = int(chunk_size)
        self.row_tile = int(row_tile)
        self.max_running = int(max_running) if max_running else self.cache.max_seqs
        self.eos = tuple(engine.spec.eos_token_ids if eos_token_ids is None else eos_token_ids)
        self.sampler = sampler if sampler is not None else Sampler(engine.rt.device, slots=self.cache.max_seqs)
        self.waiting: Deque[Request] = deque()
        self.running: List[Request] = []          # in order of admission
        self.requests: Dict[Hashable, Request] = {}
        self._ids = itertools.count()
        self._arrivals = itertools.count()
        self.steps = 0
        self.preemptions = 0
        self.last_batch_tokens = 0
        self.lookahead = bool(lookahead)
        self._inflight = None            # (PendingTokens, [(request, params)]) of the step before

    # ---- submitting -----------------------------------------------------
    def add_request(self, prompt: Sequence[int], max_new_tokens: int = 128,
                    params: Optional[SamplingParams] = None, rid: Hashable = None,
                    first_token_greedy: bool = False) -> Hashable:
        prompt = [int(t) for t in prompt]
        if not prompt:
            raise ValueError("add_request: inputs must not be empty")
        if max_new_tokens <= 0:
            max_new_tokens = 512                       # src/llaisys/models/qwen2.cpp:793
        vocab = self.engine.spec.vocab_size
        if min(prompt) < 0 or max(prompt) >= vocab:
            raise ValueError(f"add_request: a token id is outside the vocabulary of {vocab}")
        limit = self.engine.spec.max_positions
        if len(prompt) + max_new_tokens - 1 > limit:
            raise ValueError("add_request: requested prompt and output exceed model max sequence "
                             f"length ({limit})")
        need = self.cache.pages_needed(None, len(prompt) + max_new_tokens - 1, cached=0)
        for g, n in zip(self.cache.groups, need):
            if g.need.window > 0:                      # there a request goes on token by token if it must
                n = min(n, -(-g.need.window // self.cache.page_size) + 1)
            if n > g.pool.capacity:
                raise ValueError(f"add_request: the request needs {n} cache pages, the pool has "
                                 f"{g.pool.capacity}: it could never run")
        if rid is None:
            rid = next(self._ids)
            while rid in self.requests:
                rid = next(self._ids)
        elif rid in self.requests and self.requests[rid].state != FINISHED:
            raise ValueError(f"add_request: request id {rid!r} is in use")
        req = Request(rid, prompt, int(max_new_tokens), params, first_token_greedy,
                      arrival=next(self._arrivals))
        self.requests[rid] = req
        self.waiting.append(req)
        return rid

    # ---- queries -----------------------------------------------------------
    def has_unfinished(self) -> bool:
        return bool(self.waiting or self.running)

    def num_requests(self) -> int:
        return len(self.requests)

    def is_finished(self, rid) -> bool:
        return self.requests[rid].state == FINISHED

    def output(self, rid) -> List[int]:
        return list(self.requests[rid].generated)

    def abort(self, rid) -> None:
        req = self.requests[rid]
        if req.state == FINISHED:
            return
        if req.state == RUNNING:
            self.running.remove(req)
            self.engine.finish(rid)
        else:
            self.waiting.remove(req)
        req.state, req.finish_reason = FINISHED, "aborted"

    # ---- planning ------------------------------------------------------------
    def _preempt(self, req: Request) -> None:
        self.running.remove(req)
        self.engine.finish(req.rid)
        req.state, req.computed, req.bound = WAITING, 0, None
        req.preemptions += 1
        self.preemptions += 1
        self.waiting.appendleft(req)

    def _at_a_time(self, need, portion: Optional[int] = None):
        """`need` (pages per group, a list or an array [requests, groups]) counts every page that a
        request's further tokens fill.  A windowed group gives pages back as the window passes them:
        there a request holds at most the window's pages and those of the portion that a step brings
        (up to `chunk_size` tokens) at a time, and that is what has to be free for it; a pool smaller
        than that serves one request at a time, in shorter portions."""
        P = self.cache.page_size
        portion = self.chunk_size if portion is None else portion
        caps = [min(-(-(g.need.window - 1 + portion) // P) + 1, g.pool.capacity) if g.need.window > 0 else None
                for g in self.cache.groups]
        if all(c is None for c in caps):
            return need
        if isinstance(need, np.ndarray):
            need = need.copy()
            for gi, c in enumerate(caps):
                if c is not None:
                    np.minimum(need[:, gi], c, out=need[:, gi])
            return need
        return [n if c is None else min(n, c) for n, c in zip(need, caps)]

    def _fits(self, free: List[int], rid, n: int, cached: Optional[int] = None, whole: bool = False) -> Optional[List[int]]:
        """The pages that n more tokens of the request take, if they are free (else None).  `whole`:
        the n tokens will come in portions over several steps; then windowed groups count with what
        the request holds at a time, not with every page it will ever fill."""
        need = self.cache.pages_needed(rid, n, cached)
        if whole:
            need = self._at_a_time(need)
        return need if all(a <= b for a, b in zip(need, free)) else None

    def _largest_fitting(self, free: List[int], rid, n: int, cached: Optional[int]) -> int:
        """The largest portion <= n whose pages are free (0 if not even one token fits)."""
        while n > 0:
            if self._fits(free, rid, n, cached) is not None:
                return n
            have = (self.cache.cached_len(rid) if cached is None else cached) + n
            n -= ((have - 1) % self.cache.page_size) + 1        # drop the last, partly used page
        return 0

    def _end_lone(self, r: Request) -> None:
        """A request that has the pool to itself and still cannot go on."""
        self.running.remove(r)
        self.engine.finish(r.rid)
        r.state, r.finish_reason, r.pending_take = FINISHED, "error: kv capacity", None

    def plan(self) -> List[Planned]:
        """Decide the next batch.  Preempts if it must; changes nothing else."""
        while True:
            free = self.cache.free_pages()
            plan: List[Planned] = []
            budget = self.max_batch_tokens
            left = {id(r): r.remaining for r in self.running}
            movable = [r for r in self.running if left[id(r)] > 0 and not self._ends_with_pending(r)]
            short = False
            decoding = [r for r in movable if left[id(r)] == 1]
            if decoding:
                # what each of them must take for its one token, asked for in one call; in order of
                # admission, each must fit beside those before it
                need = self.cache.pages_needed_many(self.cache.handles_of([r.rid for r in decoding]),
                                                    np.ones(len(decoding), dtype=np.int32))
                fits = (np.cumsum(need, axis=0) <= np.asarray(free, dtype=np.int64)).all(axis=1)
                for i, r in enumerate(decoding):
                    if not fits[i] or budget <= 0:
                        short = not fits[i]
                        break
                    budget -= 1
                    plan.append(Planned(r, r.computed, 1, True))
                taken = need[:len(plan)].sum(axis=0) if plan else np.zeros(len(free), dtype=np.int64)
                free = [int(a - b) for a, b in zip(free, taken)]
            if short and len(self.running) > 1:
                self._preempt(self.running[-1])
                continue
            if short:                                   # a lone request that outgrew the pool
                self._end_lone(self.running[0])
                continue
            for r in movable:
                if left[id(r)] <= 1 or budget <= 0:
                    continue
                n = self._largest_fitting(free, r.rid, min(left[id(r)], self.chunk_size, budget), None)
                if n <= 0:
                    continue
                free = [a - b for a, b in zip(free, self.cache.pages_needed(r.rid, n))]
                budget -= n
                plan.append(Planned(r, r.computed, n, n == left[id(r)]))
            # Pages that the running requests' prompts will still take are spoken for: a waiting
            # request is admitted only when everything it has to compute fits what is left after
            # them (a request let in on its first portion alone would stall beside the others, each
            # holding pages and none able to finish its prompt)
            spare = self.cache.free_pages()
            slots = self.cache.free_slots()
            if self.waiting and budget > 0 and slots > 0 and len(self.running) < self.max_running:
                going = [r for r in self.running if left[id(r)] > 0]
                if going:
                    need = self._at_a_time(self.cache.pages_needed_many(
                        self.cache.handles_of([r.rid for r in going]), np.asarray([left[id(r)] for r in going], dtype=np.int32)))
                    spare = [int(a - b) for a, b in zip(spare, need.sum(axis=0))]
            while self.waiting and budget > 0 and slots > 0 and len(self.running) < self.max_running:
                r = self.waiting[0]
                whole = self._fits(spare, None, r.remaining, 0, whole=True)
                if whole is None:
                    break                               # first come first served: nobody overtakes
                # (its first portion must fit what is free in this very step, which the windowed
                # groups' pools may cut short)
                n = self._largest_fitting(free, None, min(r.remaining, self.chunk_size, budget), 0)
                if n <= 0:
                    break
                free = [a - b for a, b in zip(free, self.cache.pages_needed(None, n, cached=0))]
                self.waiting.popleft()
                r.state = RUNNING
                self.running.append(r)
                spare = [a - b for a, b in zip(spare, whole)]
                budget -= n
                slots -= 1
                plan.append(Planned(r, 0, n, n == r.remaining))
            if plan or not movable:
                return self._whole_tiles(plan)
            # requests are running, want to go on and none can (each holds pages, none is free):
            # the most recently admitted gives way
            if len(self.running) > 1:
                self._preempt(self.running[-1])
            else:
                self._end_lone(self.running[0])

    def _whole_tiles(self, plan: List[Planned]) -> List[Planned]:
        """See `row_tile`: shortens one portion, so that the step's tokens fill whole tiles."""
        tile = self.row_tile
        if tile <= 1 or not plan:
            return plan
        total = sum(p.n for p in plan)
        over = total % tile
        if total <= tile or over == 0 or over > tile // 2:
            return plan
        for i in range(len(plan) - 1, -1, -1):
            p = plan[i]
            if not p.wants_logits and p.n - over >= tile:        # a portion that stays one, and a large one
                plan[i] = Planned(p.request, p.start, p.n - over, False)
                break
        return plan

    # ---- one step ------------------------------------------------------------
    def _ends_with_pending(self, r: Request) -> bool:
        """The token that is still on its way is the request's last, whatever it is."""
        return r.pending_take is not None and (
            r.num_generated >= r.max_new_tokens
            or len(r.prompt) + r.num_generated >= self.engine.spec.max_positions)

    def step(self, default_params: Optional[SamplingParams] = None) -> List[Tuple[Hashable, int]]:
        """Plan a batch, run it, sample, finish.  Returns (request id, token)
        for every token appended in this step (with lookahead: the tokens of the
        step before, which have arrived by now)."""
        plan = self.plan()
        if not plan:
            if self._inflight is not None:
                return self._resolve()
            if self.has_unfinished() and not self.running:
                # nothing runs and the head of the queue still does not fit: it never will
                r = self.waiting.popleft()
                r.state, r.finish_reason = FINISHED, "error: kv capacity"
            return []
        entries = []
        for p in plan:
            r = p.request
            take = None
            if r.pending_take is not None and p.start + p.n == len(r.prompt) + r.num_generated:
                take = [-1] * (p.n - 1) + [r.pending_take]          # the portion ends with the pending token
            entries.append(StepEntry(r.rid, r.slice_tokens(p.start, p.n),
                                     [p.n - 1] if p.wants_logits else [], take))
        self.last_batch_tokens = sum(p.n for p in plan)
        logits = self.engine.step(entries)
        self.steps += 1
        for p in plan:
            p.request.computed += p.n
        sampled = [p.request for p in plan if p.wants_logits]
        params, counters = [], []
        for r in sampled:
            sp = r.params or default_params or SamplingParams()
            if r.first_token_greedy and not r.num_generated:
                sp = SamplingParams()
            params.append(sp)
            counters.append(r.samples_drawn)
            if not sp.greedy:
                r.samples_drawn += 1
        if not self.lookahead:
            produced: List[Tuple[Hashable, int]] = []
            if sampled:
                for r, tok in zip(sampled, self._sample(logits, sampled, params, counters, None).result()):
                    if self._append(r, int(tok)):
                        produced.append((r.rid, int(tok)))
            return produced
        handle = self._sample(logits, sampled, params, counters, self.engine.feedback) if sampled else None
        produced = self._resolve()                   # the step before; the device is busy with this one
        if handle is not None:
            for i, r in enumerate(sampled):
                if r.state != FINISHED:
                    r.pending_take = i
            self._inflight = (handle, sampled)
        return produced

    def _sample(self, logits, sampled: List[Request], params, counters, out):
        """Tokens for the rows of `logits`.  A sampler with a table on the device gets each row's state
        slot and nothing else: a request's options and stream are written there once, when it first
        samples in its slot (and again should its options change)."""
        sampler = self.sampler
        if getattr(sampler, "table", None) is None:
            if hasattr(sampler, "sample_async"):
                return sampler.sample_async(logits, params, counters, out=out) if out is not None else \
                    sampler.sample_async(logits, params, counters)
            return _Ready(sampler.sample(logits, params, counters))
        slots, greedy = [], []
        for r, sp, c in zip(sampled, params, counters):
            if sp.greedy:
                slots.append(0)
                greedy.append(True)
                continue
            if r.bound is None or r.bound[1] is not sp and r.bound[1] != sp:
                r.bound = (self.cache.slot(r.rid), sp)
                sampler.bind(r.bound[0], sp, c)
            slots.append(r.bound[0])
            greedy.append(False)
        return sampler.sample_bound_async(logits, slots, greedy, out=out)

    def _resolve(self) -> List[Tuple[Hashable, int]]:
        """The tokens of the step in flight have to be known now: wait for them and apply them."""
        if self._inflight is None:
            return []
        handle, sampled = self._inflight
        self._inflight = None
        produced = []
        for r, tok in zip(sampled, handle.result()):
            if r.state == FINISHED:                  # ended meanwhile (an end token one step back, an abort)
                continue
            r.pending_take = None
            if self._append(r, int(tok)):
                produced.append((r.rid, int(tok)))
        return produced

    def _append(self, r: Request, tok: int) -> bool:
        """Apply the finishing rules; True if the token was kept."""
        if tok in self.eos:
            self._finish(r, "eos")
            return False
        r.generated.append(tok)
        if len(r.generated) >= r.max_new_tokens:
            self._finish(r, "length")
        elif len(r.prompt) + len(r.generated) >= self.engine.spec.max_positions:
            self._finish(r, "max_pos")
        return True

    def _finish(self, r: Request, reason: str) -> None:
        r.state, r.finish_reason = FINISHED, reason
        r.pending_take = r.bound = None
        if r in self.running:
            self.running.remove(r)
        elif r in self.waiting:                      # preempted while its last token was on its way
            self.waiting.remove(r)
        self.engine.finish(r.rid)

    def run_to_completion(self, default_params: Optional[SamplingParams] = None, max_steps: int = 10 ** 9):
        while self.has_unfinished() and max_steps > 0:
            self.step(default_params)
            max_steps -= 1

"""The scheduler: which requests run in the next step, and with how many
tokens each.  Host-only; it talks to the cache manager and to nothing on a
device, so its decisions can be tested without a GPU.

Policy, after ``fastgen/generate.py:477-613`` with one change: the reference
runs a decode round and then a separate prefill phase cut every
``max_prefill`` tokens (``801-851``); here every step has one token budget,
spent first on one token for each decoding request and then on prompt
portions in arrival order, so prompt portions ride beside decoded tokens.

* Admission is first come, first served, preempted requests before new ones
  (``540-572``), while fewer than ``max_batch`` requests are live and the
  free pages hold the request's known tokens plus one.
* When a decoding request needs a page and none is free, the request admitted
  last is preempted: its pages go back, it returns to the head of the waiting
  line and is later recomputed from its prompt and everything it generated
  (``497-502``, ``772``).  A request that is alone and still out of pages ends
  there with reason ``"cache_full"`` (the reference lets it run into its
  length cap, ``509-513``).
* A request ends when it samples a stop id, has ``max_new`` tokens, or reaches
  ``max_seq`` tokens (``95-113``, ``445-447``, ``637-662``).
* The host may run one step behind the device: ``commit`` without tokens records
  a step whose samples are still on the device (a ``PENDING`` place in
  ``generated``), the next plan is made from the counts alone, and ``resolve``
  fills the values in when they arrive.  A stop id then ends its request one step
  late: what the request did in that step is dropped.
"""

from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field
from typing import Callable, Deque, Hashable, List, Optional, Sequence, Tuple

from ..cache.manager import CacheManager


PENDING = -1  # in ``Request.generated``: a token that the device has sampled and the host has not seen yet


@dataclass(eq=False)  # requests are compared by identity: two with equal fields are still two
class Request:
    rid: Hashable
    prompt: List[int]
    max_new: int
    temperature: float = 0.0
    top_p: float = 1.0
    seed: int = 0
    stop_ids: Tuple[int, ...] = ()
    want_logprobs: bool = False
    generated: List[int] = field(default_factory=list)
    logprobs: List[float] = field(default_factory=list)
    n_fed: int = 0  # tokens of prompt + generated whose keys are in the cache
    n_pending: int = 0  # PENDING places in ``generated``
    preemptions: int = 0
    finish_reason: Optional[str] = None
    # a request whose prompt and ``max_new`` tokens can never be held by the cache at once is
    # refused when it is added, unless it agrees to end early (reason ``max_seq``)
    truncate: bool = False
    keep_stop_token: bool = True  # False: a stop id that ends the request is not part of what is reported

    def all_tokens(self) -> List[int]:
        return self.prompt + self.generated

    def tokens_from(self, start: int, n: int) -> List[int]:
        """``all_tokens()[start:start+n]`` without building the whole list."""
        np_ = len(self.prompt)
        if start >= np_:
            return self.generated[start - np_ : start - np_ + n]
        if start + n <= np_:
            return self.prompt[start : start + n]
        return self.prompt[start:] + self.generated[: start + n - np_]

    def n_known(self) -> int:
        return len(self.prompt) + len(self.generated)

    def remaining(self) -> int:
        """Known tokens not yet in the cache; feeding the last one yields the
        logits of the next token."""
        return self.n_known() - self.n_fed


@dataclass(eq=False)
class PlannedEntry:
    request: Request
    start: int  # index into all_tokens()
    n: int
    wants_logits: bool  # this portion ends at the last known token
    gen_index: int = -1  # where in ``generated`` the step's sample goes (set by ``commit``)


class Scheduler:
    def __init__(self, cache: CacheManager, max_batch: int, max_step_tokens: int,
                 max_seq: Optional[int] = None, on_admit: Optional[Callable[[Hashable], None]] = None,
                 admit_reserve: int = 128) -> None:
        """``admit_reserve``: a request is admitted only while the free pages hold, beside its known
        tokens, this many more of its own and of every running request's tokens still to come (less
        where a request's cap is nearer).  The reference asks for the prompt and a 128-token buffer
        at admission (``fastgen/generate.py:535-536, 562``); with it, requests that generate up to
        128 tokens are never preempted, and longer ones rarely.  0: admit as soon as the known
        tokens and one more fit."""
        if max_batch < 1 or max_step_tokens < 1:
            raise ValueError("max_batch and max_step_tokens must be at least 1")
        if admit_reserve < 0:
            raise ValueError("admit_reserve must not be negative")
        self.admit_reserve = admit_reserve
        self.cache = cache
        self.max_batch = min(max_batch, cache.n_slots)
        self.max_step_tokens = max_step_tokens
        pool_tokens = min(cache.n_pages) * cache.page_size if cache.n_groups else 1 << 62
        self.pool_tokens = pool_tokens
        self.max_seq = min(max_seq or pool_tokens, pool_tokens)
        self._admit = on_admit or cache.admit
        self.waiting: Deque[Request] = deque()
        self.running: List[Request] = []  # in order of admission
        self.finished: List[Request] = []
        self.n_preemptions = 0
        self._served_last: Optional[Request] = None  # the last request that step A gave a token

    # ------------------------------------------------------------- intake
    def add(self, req: Request) -> None:
        if not req.prompt:
            raise ValueError(f"request {req.rid!r}: empty prompt")
        if len(req.prompt) + 1 > self.max_seq:
            raise ValueError(
                f"request {req.rid!r}: a prompt of {len(req.prompt)} tokens can never fit"
                f" (at most {self.max_seq} tokens a request)"
            )
        if req.max_new < 1:
            raise ValueError(f"request {req.rid!r}: max_new must be at least 1")
        # the reference clamps silently: maxlen = min(len + max_gen, max_seq), fastgen/generate.py:95-113
        if len(req.prompt) + req.max_new > self.pool_tokens and not req.truncate:
            raise ValueError(
                f"request {req.rid!r}: a prompt of {len(req.prompt)} tokens and {req.max_new} new ones can never"
                f" fit: the cache holds {self.pool_tokens} tokens (ask for fewer, or let it be cut short: truncate)"
            )
        self.waiting.append(req)

    def has_work(self) -> bool:
        return bool(self.waiting or self.running)

    def abort(self, rid) -> bool:
        """End the request ``rid`` now, waiting or running: its pages and slot go back and it is
        reported as ended with reason ``aborted``.  False if there is no such request."""
        for req in list(self.running) + list(self.waiting):
            if req.rid == rid:
                if req in self.waiting:
                    self.waiting.remove(req)
                self._finish(req, "aborted")
                return True
        return False

    # --------------------------------------------------------------- plan
    def _preempt(self, victim: Request) -> None:
        self.cache.release(victim.rid)
        victim.n_fed = 0
        victim.preemptions += 1
        self.n_preemptions += 1
        self.running.remove(victim)
        self.waiting.appendleft(victim)

    def _finish(self, req: Request, reason: str) -> None:
        req.finish_reason = reason
        if self.cache.is_live(req.rid):
            self.cache.release(req.rid)
        if req in self.running:
            self.running.remove(req)
        # a request preempted with a sample still on the device waits for re-admission; when that
        # sample turns out to be a stop id it must not be admitted again
        if any(r is req for r in self.waiting):
            self.waiting = deque(r for r in self.waiting if r is not req)
        self.finished.append(req)

    def _fits(self, req: Request, n: int) -> int:
        """The largest ``m <= n`` such that ``m`` more tokens of ``req`` fit in
        the pages it holds plus the free ones."""
        for g in range(self.cache.n_groups):
            held = self.cache.n_table_entries(req.rid, g)
            room = (held + self.cache.free_pages(g)) * self.cache.page_size - self.cache.length(req.rid)
            n = min(n, room)
        return max(0, n)

    def _horizon_pages(self, req: Request) -> int:
        """Pages of one group that ``req`` holds once it has grown by the admission reserve, or to its cap."""
        cap = min(len(req.prompt) + req.max_new, self.max_seq)
        tokens = max(req.n_known() + 1, min(cap, req.n_known() + self.admit_reserve))
        return -(-tokens // self.cache.page_size)

    def _promised(self) -> List[int]:
        """Per group: pages that the running requests are still expected to take (see ``admit_reserve``)."""
        out = [0] * self.cache.n_groups
        if self.admit_reserve:
            for r in self.running:
                want = self._horizon_pages(r)
                for g in range(self.cache.n_groups):
                    out[g] += max(0, want - self.cache.n_table_entries(r.rid, g))
        return out

    def plan(self) -> List[PlannedEntry]:
        entries: List[PlannedEntry] = []
        budget = self.max_step_tokens
        gone = set()  # ids of requests preempted or ended while planning
        # A. one token for every decoding request, oldest first; make room by
        #    preempting the youngest.  A budget smaller than the number of decoding
        #    requests goes round: the walk starts behind the request served last.
        walk = list(self.running)
        if budget < len(walk) and any(r is self._served_last for r in walk):
            at = next(i for i, r in enumerate(walk) if r is self._served_last) + 1
            walk = walk[at:] + walk[:at]
        for req in walk:
            if budget == 0:
                break
            if id(req) in gone or req.remaining() != 1:
                continue
            while not self.cache.can_reserve(req.rid, 1):
                victim = self.running[-1]
                if victim is req and len(self.running) == 1:
                    self._finish(req, "cache_full")
                    gone.add(id(req))
                    break
                # an entry already planned for the victim is withdrawn
                entries = [e for e in entries if e.request is not victim]
                self._preempt(victim)
                gone.add(id(victim))
                if victim is req:
                    break
            if id(req) in gone:
                continue
            self.cache.reserve(req.rid, 1)
            entries.append(PlannedEntry(req, req.n_fed, 1, True))
            self._served_last = req
            budget -= 1
        budget = self.max_step_tokens - sum(e.n for e in entries)
        planned = {id(e.request) for e in entries}
        # B. portions of prompts already admitted, oldest first
        for req in self.running:
            if budget == 0:
                break
            rem = req.remaining()
            if rem < 1 or id(req) in planned:
                continue
            n = self._fits(req, min(rem, budget))
            if n < 1:
                continue
            self.cache.reserve(req.rid, n)
            entries.append(PlannedEntry(req, req.n_fed, n, n == rem))
            budget -= n
        # C. admission: preempted requests first (they sit at the head), then new ones
        promised = self._promised() if self.waiting and len(self.running) < self.max_batch and budget > 0 else []
        while self.waiting and len(self.running) < self.max_batch and budget > 0:
            req = self.waiting[0]
            if req.n_pending:  # preempted in this very plan with a sample still on the device: next time
                break
            need = req.n_known() + 1
            if any(self.cache.pages_needed_fresh(need, g) > self.cache.free_pages(g)
                   for g in range(self.cache.n_groups)):
                break
            # with others running, room for what they and the newcomer are about to grow by as well
            own = self._horizon_pages(req)
            if self.running and self.admit_reserve and any(
                    own + promised[g] > self.cache.free_pages(g) for g in range(self.cache.n_groups)):
                break
            self.waiting.popleft()
            self._admit(req.rid)
            self.running.append(req)
            n = min(req.remaining(), budget)
            self.cache.reserve(req.rid, n)
            if self.admit_reserve:  # what it has not taken yet of its horizon is promised to it from here on
                promised = [p + max(0, own - self.cache.n_table_entries(req.rid, g)) for g, p in enumerate(promised)]
            entries.append(PlannedEntry(req, req.n_fed, n, n == req.remaining()))
            budget -= n
        # D. nothing can move although requests are live: the pages are all
        #    held by half-fed prompts; the youngest gives way
        if not entries and len(self.running) > 1:
            self._preempt(self.running[-1])
            return self.plan()
        return entries

    # -------------------------------------------------------- decode runs
    def plan_decode_run(self, max_steps: int) -> int:
        """How many decode steps all running requests can take in a row without
        the host looking at a token in between (0: take single steps).  That is
        when every running request is decoding, nobody waits for a place that a
        finishing request would free, and no request reaches its length cap or
        runs out of pages before the run ends.  (The reference runs ``sync_freq``
        steps when its batch is full, ``fastgen/generate.py:690-699``.)"""
        if max_steps < 2 or not self.running or self.waiting:
            return 0
        n = max_steps
        for req in self.running:
            if req.remaining() != 1 or req.n_pending:
                return 0
            n = min(n, req.max_new - len(req.generated), self.max_seq - req.n_known())
        if n < 2:
            return 0
        for g in range(self.cache.n_groups):
            need = sum(self.cache.pages_needed(r.rid, n)[g] for r in self.running)
            if need > self.cache.free_pages(g):
                return 0
        return n

    def commit_run(self, tokens: Sequence[Sequence[int]], logprobs: Optional[Sequence[Sequence[float]]] = None,
                   ) -> List[Request]:
        """Record a decode run: ``tokens[s][b]`` is what running request ``b``
        sampled at step ``s``.  A request that sampled a stop id ends there; what
        it sampled afterwards is dropped (``fastgen/generate.py:647-662``)."""
        done: List[Request] = []
        n = len(tokens)
        for b, req in enumerate(list(self.running)):
            req.n_fed += n
            reason = None
            for s in range(n):
                tok = int(tokens[s][b])
                req.generated.append(tok)
                if logprobs is not None and req.want_logprobs:
                    req.logprobs.append(float(logprobs[s][b]))
                if tok in req.stop_ids:
                    reason = "stop"
                elif len(req.generated) >= req.max_new:
                    reason = "length"
                elif req.n_known() >= self.max_seq:
                    reason = "max_seq"
                if reason:
                    break
            if reason:
                self._finish(req, reason)
                done.append(req)
        return done

    # ------------------------------------------------------------- commit
    def commit(self, entries: Sequence[PlannedEntry], sampled: Optional[Sequence[int]] = None,
               logprobs: Optional[Sequence[float]] = None) -> List[Request]:
        """Record what the step did: ``sampled`` holds one token for every
        entry that wanted logits, in order.  Returns the requests that ended.

        With ``sampled`` None the samples are still on the device: the places
        in ``generated`` are marked ``PENDING`` (and :meth:`resolve` fills them
        in), and only what does not depend on a token's value ends a request
        here (its count of tokens, its length)."""
        done: List[Request] = []
        i = -1
        for e in entries:
            req = e.request
            req.n_fed += e.n
            if not e.wants_logits:
                continue
            i += 1
            e.gen_index = len(req.generated)
            reason = None
            if sampled is None:
                req.generated.append(PENDING)
                req.n_pending += 1
                if req.want_logprobs:
                    req.logprobs.append(0.0)
            else:
                tok = int(sampled[i])
                req.generated.append(tok)
                if logprobs is not None and req.want_logprobs:
                    req.logprobs.append(float(logprobs[i]))
                if tok in req.stop_ids:
                    reason = "stop"
            if reason is None:
                if len(req.generated) >= req.max_new:
                    reason = "length"
                elif req.n_known() >= self.max_seq:
                    reason = "max_seq"
            if reason:
                self._finish(req, reason)
                done.append(req)
        return done

    def resolve(self, entries: Sequence[PlannedEntry], sampled: Sequence[int],
                logprobs: Optional[Sequence[float]] = None) -> List[Request]:
        """The tokens of a step that was committed without them have arrived.
        A request that sampled a stop id ends there: what it generated after
        that token (a later step may be committed already) is dropped.  Returns
        the requests that this ended."""
        late: List[Request] = []
        i = -1
        for e in entries:
            if not e.wants_logits:
                continue
            i += 1
            req = e.request
            if e.gen_index >= len(req.generated):
                continue  # dropped: the request ended on an earlier token
            if req.generated[e.gen_index] != PENDING:
                raise RuntimeError(f"request {req.rid!r}: token {e.gen_index} resolved twice")
            tok = int(sampled[i])
            req.generated[e.gen_index] = tok
            req.n_pending -= 1
            if logprobs is not None and req.want_logprobs:
                req.logprobs[e.gen_index] = float(logprobs[i])
            if tok in req.stop_ids and req.finish_reason != "aborted":
                dropped = req.generated[e.gen_index + 1:]
                req.n_pending -= sum(1 for t in dropped if t == PENDING)
                del req.generated[e.gen_index + 1:]
                del req.logprobs[e.gen_index + 1:]
                if req.finish_reason is None:
                    self._finish(req, "stop")
                    late.append(req)
                else:  # its count of tokens had ended it already: the stop id is the reason
                    req.finish_reason = "stop"
        return late

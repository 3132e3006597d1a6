"""Continuous batching above the step function.

Each round (reference: ``ServingScheduler::drive_once``, src/engine.rs:1938-1988):
  1. admit queued requests while fewer than ``max_active_sequences`` are live
     (FIFO; a request that could never fit is rejected up front, :2839-2863);
  2. visit the live requests in queue order under a token budget: a decoding request
     costs one token, a prefilling one gets ``min(prefill_token_quantum, rest of the
     prompt, budget left)`` (:2005-2095); requests not reached keep their place;
  3. run all chosen lanes as one step.  If the pages do not suffice the last lane is
     dropped and the step retried (:2145-2149); if a single lane cannot fit, that request
     alone fails with ``resource_exhausted`` and gives back what it holds (:2150-2153,
     :2205-2231).  There is no preemption or swap.  A step that fails once launched ends the
     requests of its lanes (``failed: ...``), whose pages and slots the engine has taken back;
  4. sample for the lanes whose last prompt token or decoded token ran; a cancelled request ends
     before its token is emitted, a stop token ends the request without being emitted, a
     ``False`` from the caller's ``on_token`` ends it after the token, ``max_new_tokens`` ends
     it with the token emitted (src/generation.rs:1217-1263).  A request cancelled while it
     waits never starts; one cancelled between rounds gives back what it holds before the next
     (src/engine.rs:1136-1143, 1668-1672, 1753-1765);
  5. finished requests give back pages and slot; visited ones go to the back of the line.

One round ahead.  With a sampler that can leave its tokens on the device (``sample_async``) and an engine that
can take a lane's token from there (``feeds_tokens``), a round is queued on the GPU before the tokens of the
round before it have reached the host: a decoding request's lane is fed from the device, and the host reads
the earlier round's tokens (emits them, applies the stop conditions) while the GPU works.  A request that
turns out to have ended in the earlier round (a stop token, the caller's ``on_token``, a cancellation) has
then run one token too far: that token is dropped and what the request held is given back as usual; a request
that ends by ``max_new_tokens`` is known beforehand and is not queued again.  Penalties count the token that
is still on the device there.  With a sampler or an engine that cannot do this every round waits for its
tokens (as the reference does, src/engine.rs:1938-1988).
"""
from __future__ import annotations

import time
from collections import deque
from dataclasses import dataclass, field
from typing import Callable, Deque, Dict, Hashable, List, Optional, Sequence

from ..cache.pages import CacheExhausted
from ..sampling.params import SamplingParams
from ..sampling.sampler import SamplerRow
from .context import Lane
from .engine import StepFailed


@dataclass
class EngineConfig:
    """Scheduler knobs, with the reference's names (src/engine.rs:309-385).  The reference's
    defaults (2 / 256 / 128 / 8) are sized for a laptop; these are sized for one MI355X."""
    max_active_sequences: int = 64
    scheduler_token_budget: int = 4096
    prefill_token_quantum: int = 2048
    queue_capacity: int = 4096

    def __post_init__(self):
        if min(self.max_active_sequences, self.scheduler_token_budget, self.prefill_token_quantum,
               self.queue_capacity) <= 0:
            raise ValueError("scheduler settings must be positive")
        if self.prefill_token_quantum > self.scheduler_token_budget:
            raise ValueError("prefill_token_quantum cannot exceed scheduler_token_budget")


@dataclass
class Request:
    request_id: Hashable
    prompt: List[int]
    params: SamplingParams
    generated: List[int] = field(default_factory=list)
    cursor: int = 0                        # prompt tokens already in the cache
    finish_reason: Optional[str] = None    # "stop", "length", "cancelled", "resource_exhausted", "rejected: ..."
    cancelled: bool = False
    submitted_at: float = 0.0
    started_at: Optional[float] = None     # admission: the request got its slot
    first_token_at: Optional[float] = None
    finished_at: Optional[float] = None
    in_flight: Optional[tuple] = None      # (tokens still on the device, this request's row among them)

    @property
    def finished(self) -> bool:
        return self.finish_reason is not None

    @property
    def prefilling(self) -> bool:
        return self.cursor < len(self.prompt)

    def cancel(self) -> None:
        """Ask for the request to end; the scheduler honours it at its next decision about it."""
        self.cancelled = True


class QueueFull(RuntimeError):
    pass


class Scheduler:
    def __init__(self, engine, sampler, config: Optional[EngineConfig] = None,
                 stop_token_ids: Sequence[int] = (), on_token: Optional[Callable] = None):
        """``engine``: add_request / finish / step(lanes) / cache.can_ever_fit / vocab_size /
        max_context.  ``sampler``: sample(logits, rows) -> tokens.  ``on_token(request, token)`` is
        called for every emitted token; returning ``False`` ends that request there (its own stop
        condition), ``request.cancel()`` ends it before its next token."""
        self.engine = engine
        self.sampler = sampler
        self.config = config or EngineConfig()
        self.stop_token_ids = set(int(token) for token in stop_token_ids)
        self.on_token = on_token
        self.queue: Deque[Request] = deque()
        self.active: Deque[Request] = deque()
        self.finished: Dict[Hashable, Request] = {}
        self.rounds = 0
        self.last_lanes: List[Lane] = []        # what the last round ran (for tests and metrics)
        self.ahead = (getattr(sampler, "sample_async", None) is not None
                      and bool(getattr(engine, "feeds_tokens", False)))
        self._pending: Optional[tuple] = None   # (tokens on their way to the host, the requests they are for)

    # ------------------------------------------------------------------ submission
    def submit(self, request_id: Hashable, prompt: Sequence[int], params: SamplingParams) -> Request:
        if len(self.queue) >= self.config.queue_capacity:
            raise QueueFull(f"the queue holds {len(self.queue)} requests, its capacity")
        request = Request(request_id, [int(token) for token in prompt], params, submitted_at=time.perf_counter())
        self.queue.append(request)
        return request

    def has_work(self) -> bool:
        return bool(self.queue or self.active or self._pending)

    def cancel(self, request_id: Hashable) -> bool:
        """Cancel a waiting or live request; False if there is no such request (any more)."""
        for request in list(self.queue) + list(self.active):
            if request.request_id == request_id:
                request.cancel()
                return True
        return False

    # ------------------------------------------------------------------ one round
    def _reject(self, request: Request, why: str) -> None:
        request.finish_reason = f"rejected: {why}"
        request.finished_at = time.perf_counter()
        self.finished[request.request_id] = request

    def _admit(self) -> None:
        for request in [request for request in self.active if request.cancelled]:
            self._finish(request, "cancelled")
        while self.queue and len(self.active) < self.config.max_active_sequences:
            request = self.queue.popleft()
            needed = len(request.prompt) + request.params.max_new_tokens - 1
            if request.cancelled:                      # never starts, holds nothing
                request.finish_reason = "cancelled"
                request.finished_at = time.perf_counter()
                self.finished[request.request_id] = request
            elif not request.prompt:
                self._reject(request, "prompt must contain at least one token")
            elif any(not (0 <= token < self.engine.vocab_size) for token in request.prompt):
                self._reject(request, "input contains a token ID outside the model vocabulary")
            elif (isinstance(request.params.allowed_token_ids, tuple)
                  and max(request.params.allowed_token_ids) >= self.engine.vocab_size):
                self._reject(request, "allowed_token_ids names a token ID outside the model vocabulary")
            elif needed > self.engine.max_context:
                self._reject(request, "prompt plus requested output exceeds model context limit")
            elif not self.engine.cache.can_ever_fit(needed):
                self._reject(request, "prompt plus requested output exceeds the cache capacity")
            else:
                self.engine.add_request(request.request_id)
                request.started_at = time.perf_counter()
                self.active.append(request)

    def _collect(self) -> List[tuple]:
        """(request, tokens, samples?) for this round, in queue order under the budget."""
        budget = self.config.scheduler_token_budget
        visits = []
        for request in self.active:
            if budget <= 0:
                break
            if request.prefilling:
                count = min(self.config.prefill_token_quantum, len(request.prompt) - request.cursor, budget)
                tokens = request.prompt[request.cursor:request.cursor + count]
                samples = request.cursor + count == len(request.prompt)
            elif request.in_flight is not None:
                if len(request.generated) + 1 >= request.params.max_new_tokens:
                    continue                              # the token on its way is its last one
                tokens = [0]                              # stands for the token that is still on the device
                samples = True
            else:
                tokens = [request.generated[-1]]
                samples = True
            budget -= len(tokens)
            visits.append((request, tokens, samples))
        return self._trim(visits)

    def _trim(self, visits: List[tuple]) -> List[tuple]:
        """An engine that runs steps of certain sizes best says so (``step_token_target``): a portion that does
        not end its prompt anyway is cut shorter by the few tokens that make the step such a size."""
        target = getattr(self.engine, "step_token_target", None)
        if target is None or not visits:
            return visits
        total = sum(len(tokens) for _, tokens, _ in visits)
        lanes = len(visits)
        # an engine that runs the single tokens of a step as a batch of their own sizes the portions without them
        singles = sum(1 for _, tokens, _ in visits if len(tokens) == 1)
        split_from = getattr(self.engine, "split_from_lanes", None)
        if split_from is not None and split_from <= singles < lanes:
            lanes, total = lanes - singles, total - singles
        for index in range(len(visits) - 1, -1, -1):
            request, tokens, samples = visits[index]
            if request.prefilling and not samples and len(tokens) > 1:
                spare = total - int(target(lanes, total))
                if 0 < spare < len(tokens):
                    visits[index] = (request, tokens[:len(tokens) - spare], False)
                break
        return visits

    def _finish(self, request: Request, reason: str, release: bool = True) -> None:
        request.finish_reason = reason
        request.finished_at = time.perf_counter()
        if release:
            self.engine.finish(request.request_id)
        self.active.remove(request)
        self.finished[request.request_id] = request

    def _resolve(self, pending: Optional[tuple] = None) -> None:
        """Wait for a round's tokens and do with them what step 4 says."""
        if pending is None:
            pending, self._pending = self._pending, None
        if pending is None:
            return
        handle, requests = pending
        tokens_out = handle.wait()
        now = time.perf_counter()
        for request, token in zip(requests, tokens_out):
            if request.in_flight is not None and request.in_flight[0] is handle:
                request.in_flight = None
            if not request.finished:                 # else it ended a round earlier: one token too far, dropped
                self._complete(request, int(token), now)

    def _needs_tokens_first(self) -> bool:
        """Whether the round before has to be read before the next can be made up."""
        if self._pending is None:
            return False
        return not self.ahead

    def step(self) -> List[Request]:
        """One round; returns the requests that finished in it."""
        self.rounds += 1
        done_before = set(self.finished)
        if self._needs_tokens_first():
            self._resolve()
        self._admit()
        visits = self._collect()
        logits = None
        while visits:
            lanes = [Lane(request.request_id, tokens, [len(tokens) - 1] if samples else [],
                          feed=(request.in_flight[0].device, request.in_flight[1])
                          if request.in_flight is not None and not request.prefilling else None)
                     for request, tokens, samples in visits]
            try:
                logits = self.engine.step(lanes)
                self.last_lanes = lanes
                break
            except CacheExhausted:
                if len(visits) > 1:
                    visits.pop()                 # the last lane waits for a later round
                elif self._pending is not None:
                    # a round is still on its way: its tokens may end requests (this one too) and give pages
                    # back, so they are read first and the round is made up again from what is then live
                    self._resolve()
                    visits = self._collect()
                else:
                    self._finish(visits[0][0], "resource_exhausted")
                    visits = self._collect()
            except StepFailed as failure:
                # the engine has ended the step's requests and taken back what they held; the others go on
                self._resolve()
                for request, _, _ in visits:
                    if not request.finished:
                        self._finish(request, f"failed: {failure.__cause__}", release=False)
                visits = []
        before, self._pending = self._pending, None
        if visits:
            sampled = [(request, tokens) for request, tokens, samples in visits if samples]
            for request, tokens, samples in visits:
                if request.prefilling:
                    request.cursor += len(tokens)
            if sampled and before is not None and any(request.params.constrained_by_history for request, _ in sampled):
                # a constraint that reads what was generated: the round on its way is read first (the GPU works
                # on this round's forward pass meanwhile); a request that it ended drops out of the sampling
                self._resolve(before)
                before = None
                keep = [row for row, (request, _) in enumerate(sampled) if not request.finished]
                if len(keep) < len(sampled):
                    sampled = [sampled[row] for row in keep]
                    logits = logits[keep] if keep else None
            if sampled:
                rows, kept = [], []
                for row, (request, _) in enumerate(sampled):
                    try:
                        made = SamplerRow(request.params, request.prompt, request.generated,
                                          None if request.in_flight is None
                                          else (request.in_flight[0].device, request.in_flight[1]))
                        if made.allowed is not None and max(made.allowed) >= self.engine.vocab_size:
                            raise ValueError("the constraint names a token ID outside the model vocabulary")
                        rows.append(made)
                        kept.append(row)
                    except Exception as error:           # its constraint allows no token, or fails itself: the request fails alone
                        self._finish(request, f"failed: {error}")
                if len(kept) < len(sampled):
                    sampled = [sampled[row] for row in kept]
                    logits = logits[kept] if kept else None
            if sampled:
                if self.ahead:
                    handle = self.sampler.sample_async(logits, rows)
                    self._pending = (handle, [request for request, _ in sampled])
                else:
                    tokens_out = self.sampler.sample(logits, rows)
                    now = time.perf_counter()
                    for (request, _), token in zip(sampled, tokens_out):
                        self._complete(request, int(token), now)
        if before is not None:
            self._resolve(before)                # the GPU works on this round meanwhile
        if self._pending is not None:
            for row, request in enumerate(self._pending[1]):
                request.in_flight = (self._pending[0], row)
        if visits:
            for request, _, _ in visits:         # visited requests go to the back of the line
                if not request.finished:
                    self.active.remove(request)
                    self.active.append(request)
        return [request for key, request in self.finished.items() if key not in done_before]

    def _complete(self, request: Request, token: int, now: float) -> None:
        params = request.params
        if request.cancelled:                        # before the token becomes visible
            self._finish(request, "cancelled")
            return
        stops = self.stop_token_ids | set(params.stop_token_ids)
        if not params.ignore_eos and token in stops:
            self._finish(request, "stop")            # the stop token is not emitted
            return
        if request.first_token_at is None:
            request.first_token_at = now
        request.generated.append(token)
        if self.on_token is not None and self.on_token(request, token) is False:
            self._finish(request, "stop")            # the caller's own stop condition; the token stays emitted
        elif len(request.generated) >= params.max_new_tokens:
            self._finish(request, "length")

    def run(self, on_round: Optional[Callable] = None) -> Dict[Hashable, Request]:
        """Rounds until every submitted request has finished; ``on_round(seconds)`` after each."""
        while self.has_work():
            started = time.perf_counter()
            self.step()
            if on_round is not None:
                on_round(time.perf_counter() - started)
        return self.finished

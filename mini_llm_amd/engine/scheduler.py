"""Continuous batching over the step function.

The reference's scheduler (pytorch/src/mini_llm/scheduler.py) admits a waiting request when a
cache is free, prefills its whole prompt in a call of its own, and decodes all running requests
in one batched step. This one keeps its queues, its finish reasons and their order, its error
scopes and its statistics, and differs where the engine below differs: prompts are cut into
portions under a token budget and run in the same step as the decodes, the currency of
admission is pages, and a decision is made for the case that pages run out.

Every iteration (`step`):
1. cancelled requests leave;
2. plan: running requests past their prompt bring one token each; what is left of the token
   budget goes to prompts, first those already running, then newly admitted ones in arrival
   order (no request overtakes the head of the queue; a request is admitted when the pages for
   its whole prompt are free, though it is fed in portions);
3. when pages run out for a running request, the request admitted last is preempted: it gives
   everything back and returns to the FRONT of the queue with its prompt extended by what it has
   generated, to be recomputed when there is room. A request that does not fit an empty pool
   fails;
4. one step of the engine; each request whose prompt is complete gets one new token, sampled
   on the device; `emit(token, finish)`; a finished request leaves at once and frees its pages.

One step ahead (an executor with `launch` / `collect`): the step planned in 2 is launched before
the tokens of the step before it have been read. A request that was sampled in the step in
flight brings "the token in my slot" (the sampler leaves it there on the device), so planning,
batch layout and launch of step n+1 take place while the device still runs step n, and the device
never waits for the host. What the host cannot know yet is whether token n was the request's end
token: ends by length and context are counted ahead and never launched, an end token is seen one
step late, and the one token computed past it is dropped. A finished request's pages go back at
once all the same: everything the device does is in launch order, so whoever gets them next writes
them after the step in flight has. A plan that would have to preempt first waits for the step in
flight, so that a victim's tokens are all known.
"""

from __future__ import annotations

import collections
import logging
import threading
from dataclasses import dataclass, field
from typing import Callable, Literal, Protocol

from ..sampling import SamplingParams
from .batch import StepEntry

logger = logging.getLogger(__name__)

FinishReason = Literal["stop", "length", "context"]


class StepExecutor(Protocol):
    """What the scheduler needs from the engine below it."""

    page_size: int

    def max_positions(self) -> int | None: ...
    def check_prompt(self, tokens: list[int]) -> None: ...          # raises if it can never run
    def can_open(self) -> bool: ...
    def open(self, request_id) -> None: ...
    def close(self, request_id) -> None: ...
    def length(self, request_id) -> int: ...
    def pages_needed(self, request_id, n_new: int) -> list[int]: ...  # per layer group, for its next n_new tokens
    def free_pages(self) -> list[int]: ...                            # per layer group
    def run(self, entries: list, sampling: list, steps: list) -> list[int]: ...
    # Optional, for running one step ahead: launch() queues the step and leaves each sampled token
    # in its request's last-token slot; collect() waits for that step and returns its tokens. An
    # entry with from_slot=True takes its one token from the request's slot.
    # def launch(self, entries, sampling, steps) -> object: ...
    # def collect(self, handle) -> list[int]: ...


@dataclass(eq=False)
class Request:
    """The reference's Request (scheduler.py:41-53) plus how to sample."""

    tokens: list
    max_new_tokens: int | None
    eos_token_id: int | None
    # emit(token, finish): finish is None for every token but the last one.
    emit: Callable[[int, FinishReason | None], None]
    fail: Callable[[str], None]
    sampling: SamplingParams = field(default_factory=SamplingParams)
    cancelled: bool = field(default=False, init=False)

    def cancel(self) -> None:
        self.cancelled = True


@dataclass(eq=False)  # compared by identity: membership tests must not walk every field
class _Running:
    request: Request
    request_id: int
    pending: list              # tokens not yet fed: the rest of the prompt, or the last sampled token
    history: list = field(default_factory=list)   # tokens fed since it was (re)admitted: what its pages hold
    generated: int = 0         # tokens delivered
    launched: int = 0          # tokens whose sampling has been launched (= generated, or one more)
    awaiting: bool = False     # its next token is the output of the step in flight
    fed_ahead: bool = False    # the step in flight takes the token of the step before it from the slot
    prompt_len: int = 0        # of the original prompt (a preempted request's recompute does not count)
    order: int = 0             # admission order; the largest is preempted first
    finished: bool = False


class _PagePlan:
    """Pages the step being planned has claimed so far, against what is free, per layer group."""

    def __init__(self, free):
        self.free = list(free)
        self.taken = [0] * len(self.free)

    def fits(self, need) -> bool:
        return all(t + n <= f for t, n, f in zip(self.taken, need, self.free))

    def take(self, need) -> None:
        self.taken = [t + n for t, n in zip(self.taken, need)]


@dataclass
class _Flight:
    """A step that has been launched and whose tokens have not been read."""

    handle: object
    sampled: list              # the _Running of each token, in the step's order


class _SettleFirst(Exception):
    """The plan has to preempt: the step in flight is collected first."""


class Scheduler:
    def __init__(self, executor: StepExecutor, max_batch: int = 16, max_tokens_per_step: int = 2048,
                 max_prefills_per_step: int | None = None, step_ahead: bool = True):
        if max_batch < 1 or max_tokens_per_step < 1:
            raise ValueError("max_batch and max_tokens_per_step must be at least 1")
        if max_prefills_per_step is not None and max_prefills_per_step < 1:
            raise ValueError("max_prefills_per_step must be at least 1")
        self._executor = executor
        self._max_batch, self._budget, self._max_prefills = max_batch, max_tokens_per_step, max_prefills_per_step
        self._step_ahead = step_ahead and hasattr(executor, "launch") and hasattr(executor, "collect")
        self._in_flight: _Flight | None = None
        self._waiting: collections.deque = collections.deque()   # Request, or _Running that was preempted
        self._running: list[_Running] = []
        self._wake = threading.Condition()
        self._stopping = False
        self._thread: threading.Thread | None = None
        self._next_id = 0
        self._order = 0
        self._steps = self._decode_steps = self._tokens = self._prefills = 0
        self._batch_sizes = self._step_tokens = self._preemptions = self._dropped_tokens = 0

    # --- called from other threads -------------------------------------------------------------
    def submit(self, request: Request) -> None:
        with self._wake:
            self._waiting.append(request)
            self._wake.notify()

    def stats(self) -> dict:
        steps = self._decode_steps
        return {
            "decode_steps": steps,
            "tokens": self._tokens,
            "prefills": self._prefills,
            "mean_batch_size": self._batch_sizes / steps if steps else 0.0,
            "running": len(self._running),
            "waiting": len(self._waiting),
            "steps": self._steps,
            "tokens_per_step": self._step_tokens / self._steps if self._steps else 0.0,
            "preemptions": self._preemptions,
            "dropped_tokens": self._dropped_tokens,   # computed past an end token nobody had seen yet
        }

    def start(self) -> None:
        self._thread = threading.Thread(target=self._loop, name="scheduler", daemon=True)
        self._thread.start()

    def stop(self) -> None:
        with self._wake:
            self._stopping = True
            self._wake.notify()
        if self._thread is not None:
            self._thread.join()
        self._fail_everything("the engine is shutting down")

    def is_running(self) -> bool:
        return self._thread is not None and self._thread.is_alive()

    def has_work(self) -> bool:
        with self._wake:
            return bool(self._running) or bool(self._waiting) or self._in_flight is not None

    def run_until_idle(self) -> None:
        while self.step():
            pass

    # --- the scheduler thread ------------------------------------------------------------------
    def _loop(self) -> None:
        while True:
            with self._wake:
                while not self._stopping and not self._running and not self._waiting and self._in_flight is None:
                    self._wake.wait()
                if self._stopping:
                    return
            self.step()

    def step(self) -> bool:
        """One iteration. Returns False if there was nothing to do."""
        try:
            self._drop_cancelled()
            try:
                entries, owners = self._plan()
            except _SettleFirst:
                self._collect()
                entries, owners = self._plan()
            launched = self._launch(entries, owners) if entries else None
            self._collect()                 # the step launched before this one
            self._in_flight = launched
            if not self._step_ahead:
                self._collect()
        except Exception as error:  # the engine is shared: every running request is affected
            logger.exception("engine error")
            self._fail_running(str(error))
            return True
        return bool(entries) or self.has_work()

    # --- planning ------------------------------------------------------------------------------
    def _drop_cancelled(self) -> None:
        for running in [r for r in self._running if r.request.cancelled]:
            self._executor.close(running.request_id)
            self._running.remove(running)
            running.finished = True   # a token of its that is still in flight is dropped

    def _portion_that_fits(self, running: _Running, plan: "_PagePlan", most: int):
        """(n, pages): the largest portion n <= most whose pages can be had beside what is planned
        already, and those pages per group; n = 0 if not even one token fits."""
        n = most
        while n >= 1:
            need = self._executor.pages_needed(running.request_id, n)
            if plan.fits(need):
                return n, need
            # shrink to the end of the page before the last one the portion touches
            length = self._executor.length(running.request_id)
            page = self._executor.page_size
            n = min(n - 1, ((length + n - 1) // page) * page - length)
        return 0, None

    def _preempt(self, victim: _Running) -> None:
        """The victim gives everything back and waits at the front of the queue; what it has been
        fed so far becomes prompt again, so that it is recomputed and goes on where it was."""
        assert not victim.awaiting, "a victim's tokens are all known"
        self._executor.close(victim.request_id)
        self._running.remove(victim)
        victim.pending = victim.history + victim.pending
        victim.history = []
        self._preemptions += 1
        with self._wake:
            self._waiting.appendleft(victim)

    def _plan(self):
        entries, owners = [], []
        plan = _PagePlan(self._executor.free_pages())
        budget = self._budget
        preempted = False
        # Running requests first, in admission order: decodes bring one token, prompts a portion.
        # Requests are planned oldest first and preempted youngest first, so a victim never has
        # an entry in the plan yet.
        for running in sorted(self._running, key=lambda r: r.order):
            if running not in self._running:
                continue  # preempted while an older request was planned
            if budget < 1:
                break
            if self._ends_in_flight(running):
                continue
            most = min(self._to_feed(running), budget)
            n, need = self._portion_that_fits(running, plan, most)
            while n == 0:
                if self._in_flight is not None:
                    raise _SettleFirst()   # nothing has been changed so far
                victim = max(self._running, key=lambda r: r.order)
                preempted = True
                if victim is running:
                    if len(self._running) == 1:
                        # alone, with every other page free, and still no room
                        self._executor.close(running.request_id)
                        self._running.remove(running)
                        running.request.fail("the request needs more cache pages than the pool has")
                    else:
                        self._preempt(running)
                    break
                self._preempt(victim)
                plan.free = self._executor.free_pages()
                n, need = self._portion_that_fits(running, plan, most)
            if n == 0:
                continue
            self._add_entry(entries, owners, plan, running, n, need)
            budget -= n
        # Then admissions, in arrival order; the head of the queue is never overtaken. None in a
        # step that had to preempt: the preempted request would come straight back.
        admitted = 0
        while not preempted and budget >= 1 and len(self._running) < self._max_batch:
            if self._max_prefills is not None and admitted >= self._max_prefills:
                break
            item = self._pop_waiting()
            if item is None:
                break
            running = self._admit(item, plan, bool(entries))
            if running is None:
                continue          # cancelled or failed: the next one gets its turn
            if running is False:
                self._push_front(item)
                break             # no room yet: wait for a running request to end
            n, need = self._portion_that_fits(running, plan, min(len(running.pending), budget))
            self._add_entry(entries, owners, plan, running, n, need)
            budget -= n
            admitted += 1
        return entries, owners

    @staticmethod
    def _to_feed(running: _Running) -> int:
        return 1 if running.awaiting else len(running.pending)

    def _ends_in_flight(self, running: _Running) -> bool:
        """The token being sampled in the step in flight is this request's last, whatever it is."""
        if not running.awaiting:
            return False
        request, limit = running.request, self._executor.max_positions()
        return ((limit is not None and running.prompt_len + running.launched >= limit)
                or (request.max_new_tokens is not None and running.launched >= request.max_new_tokens))

    def _add_entry(self, entries, owners, plan, running, n, need) -> None:
        if running.awaiting:
            entry = StepEntry(running.request_id, [0], [0], from_slot=True)
        else:
            completes = n == len(running.pending)
            entry = StepEntry(running.request_id, list(running.pending[:n]), [n - 1] if completes else [])
        entries.append(entry)
        owners.append(running)
        plan.take(need)

    def _admit(self, item, plan, others_planned: bool):
        """None: the request is gone (cancelled / failed). False: no room now. Else the _Running."""
        request = item.request if isinstance(item, _Running) else item
        if request.cancelled:
            return None
        if isinstance(item, _Running):
            running = item
        else:
            try:
                if not request.tokens:
                    raise ValueError("the prompt has no tokens")
                self._executor.check_prompt(list(request.tokens))
            except Exception as error:  # a bad prompt is the problem of this request only
                logger.warning("request refused: %s", error)
                request.fail(str(error))
                return None
            running = _Running(request, -1, list(request.tokens), prompt_len=len(request.tokens))
        if not self._executor.can_open():
            return False
        request_id = self._next_id
        self._executor.open(request_id)
        # Admitted only if its whole prompt has room beside what is planned: a request that could
        # take a first portion and then stall would only be preempted again.
        if not plan.fits(self._executor.pages_needed(request_id, len(running.pending))):
            self._executor.close(request_id)
            if not self._running and not others_planned:
                request.fail("the request needs more cache pages than the pool has")
                return None
            return False
        self._next_id += 1
        running.request_id = request_id
        running.order = self._order
        self._order += 1
        self._running.append(running)
        return running

    def _pop_waiting(self):
        with self._wake:
            return self._waiting.popleft() if self._waiting else None

    def _push_front(self, item) -> None:
        with self._wake:
            self._waiting.appendleft(item)

    # --- running and delivering ----------------------------------------------------------------
    def _launch(self, entries, owners) -> _Flight:
        sampled = [o for o, e in zip(owners, entries) if e.want]
        sampling = [o.request.sampling for o in sampled]
        steps = [o.launched for o in sampled]
        if self._step_ahead:
            handle = self._executor.launch(entries, sampling, steps)
        else:
            handle = self._executor.run(entries, sampling, steps)
        self._steps += 1
        self._step_tokens += sum(len(e.tokens) for e in entries)
        decodes = sum(1 for o, e in zip(owners, entries) if o.launched > 0 and len(e.tokens) == 1)
        if decodes:
            self._decode_steps += 1
            self._batch_sizes += decodes
        for owner, entry in zip(owners, entries):
            if entry.from_slot:
                owner.fed_ahead = True     # the token joins its history when it is known
            else:
                owner.history.extend(entry.tokens)
                del owner.pending[: len(entry.tokens)]
        for owner in sampled:
            owner.launched += 1
            owner.awaiting = True
        return _Flight(handle, sampled)

    def _collect(self) -> None:
        """Reads the tokens of the step in flight, if there is one, and delivers them."""
        flight, self._in_flight = self._in_flight, None
        if flight is None:
            return
        tokens = self._executor.collect(flight.handle) if self._step_ahead else flight.handle
        for owner, token in zip(flight.sampled, tokens):
            if owner.finished:
                self._dropped_tokens += 1
                continue
            token = int(token)
            if owner.generated == 0:
                self._prefills += 1
            owner.generated += 1
            if owner.fed_ahead:            # the step launched after this one has been fed it already
                owner.history.append(token)
                owner.fed_ahead = False
            else:
                owner.awaiting = False
                owner.pending = [token]
            self._deliver(owner, token)
        self._running = [r for r in self._running if not r.finished]

    def _finish_reason(self, running: _Running, token: int) -> FinishReason | None:
        # the order of the reference's checks (scheduler.py:185-196)
        request = running.request
        if request.eos_token_id is not None and token == request.eos_token_id:
            return "stop"
        limit = self._executor.max_positions()
        if limit is not None and running.prompt_len + running.generated >= limit:
            return "context"
        if request.max_new_tokens is not None and running.generated >= request.max_new_tokens:
            return "length"
        return None

    def _deliver(self, running: _Running, token: int) -> None:
        """Hands one token to its request. If that ends the request, its pages are given back."""
        reason = self._finish_reason(running, token)
        self._tokens += 1
        try:
            running.request.emit(token, reason)
        except Exception:
            # The consumer is gone. That is the problem of this request only.
            logger.exception("emit failed, dropping the request")
            reason = "stop"
        if reason is not None:
            self._executor.close(running.request_id)
            running.finished = True

    def _fail_running(self, message: str) -> None:
        running, self._running = self._running, []
        self._in_flight = None
        for item in running:
            item.finished = True
            try:
                self._executor.close(item.request_id)
            except Exception:
                logger.exception("closing a request after an engine error failed")
            item.request.fail(message)

    def _fail_everything(self, message: str) -> None:
        self._fail_running(message)
        while (item := self._pop_waiting()) is not None:
            (item.request if isinstance(item, _Running) else item).fail(message)

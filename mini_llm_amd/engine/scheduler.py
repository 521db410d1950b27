"""Continuous batching over the step function.

What is kept of the reference's scheduler (pytorch/src/mini_llm/scheduler.py) is its behaviour:
first come, first served; a request that finds no room keeps its place; the three reasons to
finish and the order in which they are looked at (:185-196); the finishing token is delivered;
an error of the engine ends every live request, a bad prompt or a failing consumer only its own
(:131-141, :170-177, :202-211); the counters of ``stats`` (:93-102). What differs follows from the
engine below: prompts are cut into portions under a token budget and run in the same step as the
decodes, admission is paid in pages, and there is a decision for the case that pages run out.
The scheduler is single-threaded: whoever calls ``step`` owns it (``engine.background`` has a
thread for callers that want one).

One iteration (``step``):
1. cancelled requests leave;
2. plan: live requests past their prompt bring one token each; what is left of the token
   budget goes to prompts, first those already live, then newly admitted ones in arrival
   order (no request overtakes the head of the queue; a request is admitted when the pages for
   its whole prompt are free, though it is fed in portions);
3. when pages run out for a live request, the request admitted last is preempted: it gives
   everything back and returns to the FRONT of the queue with its prompt extended by what it has
   generated, to be recomputed when there is room. A request that does not fit an empty pool
   fails;
4. one step of the engine; each request whose prompt is complete gets one new token, sampled
   on the device, and hears of it through ``on_token(token, finish)``; a finished request leaves
   at once and frees its pages.

One step ahead (an executor with ``launch`` / ``collect``): the step planned in 2 is launched before
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
from typing import Protocol

from ..sampling import SamplingParams
from .batch import StepEntry

log = logging.getLogger(__name__)

# Why a request ended, in the order the checks are made.
STOP, CONTEXT, LENGTH = "stop", "context", "length"


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


class Request:
    """A prompt to continue and where its tokens go.

    ``on_token(token, finish)`` is called once per generated token; ``finish`` is None except
    with the last one, where it is "stop" (the end token came, and is delivered), "context" (the
    model's positions are used up) or "length" (``max_new_tokens`` reached). ``on_error(message)``
    is called instead if the request cannot run or the engine fails under it. ``max_new_tokens``
    None: until one of the other two reasons ends it."""

    __slots__ = ("prompt", "on_token", "on_error", "max_new_tokens", "eos_token_id", "sampling", "_cancelled")

    def __init__(self, prompt, *, on_token, on_error, max_new_tokens=None, eos_token_id=None, sampling: SamplingParams | None = None):
        self.prompt = prompt
        self.on_token, self.on_error = on_token, on_error
        self.max_new_tokens, self.eos_token_id = max_new_tokens, eos_token_id
        self.sampling = SamplingParams() if sampling is None else sampling
        self._cancelled = False

    def cancel(self) -> None:
        """May be called from any thread; the scheduler looks at it before its next step."""
        self._cancelled = True

    @property
    def cancelled(self) -> bool:
        return self._cancelled


class _Live:
    """A request that holds pages. Compared by identity."""

    __slots__ = ("request", "request_id", "pending", "history", "generated", "launched", "awaiting", "fed_ahead",
                 "prompt_len", "order", "finished")

    def __init__(self, request: Request, prompt: list):
        self.request = request
        self.request_id = -1
        self.pending = prompt        # tokens not yet fed: the rest of the prompt, or the last sampled token
        self.history = []            # tokens fed since it was (re)admitted: what its pages hold
        self.generated = 0           # tokens delivered
        self.launched = 0            # tokens whose sampling has been launched (= generated, or one more)
        self.awaiting = False        # its next token is the output of the step in flight
        self.fed_ahead = False       # the step in flight takes the token of the step before it from the slot
        self.prompt_len = len(prompt)  # of the original prompt (a preempted request's recompute does not count)
        self.order = 0               # admission order; the largest is preempted first
        self.finished = False


class _PagePlan:
    """Pages the step being planned has claimed so far, against what is free, per layer group."""

    def __init__(self, free):
        self.free = list(free)
        self.taken = [0] * len(self.free)

    def fits(self, need) -> bool:
        return all(t + n <= f for t, n, f in zip(self.taken, need, self.free))

    def take(self, need) -> None:
        self.taken = [t + n for t, n in zip(self.taken, need)]


class _Flight:
    """A step that has been launched and whose tokens have not been read."""

    __slots__ = ("handle", "sampled")

    def __init__(self, handle, sampled):
        self.handle, self.sampled = handle, sampled   # sampled: the _Live of each token, in the step's order


class _SettleFirst(Exception):
    """The plan has to preempt: the step in flight is collected first."""


class _Tally:
    """Running totals behind ``stats``."""

    def __init__(self):
        self.steps = self.step_tokens = 0              # every step, and the tokens it was fed
        self.decode_steps = self.decode_rows = 0       # steps with at least one decoded token, and those tokens
        self.delivered = self.first_tokens = 0         # tokens handed out; requests that got their first one
        self.preemptions = self.dropped = 0


class Scheduler:
    NO_ROOM = "the request needs more cache pages than the pool has"

    def __init__(self, executor: StepExecutor, max_batch: int = 16, max_tokens_per_step: int = 2048,
                 max_prefills_per_step: int | None = None, step_ahead: bool = True):
        for name, value in (("max_batch", max_batch), ("max_tokens_per_step", max_tokens_per_step)):
            if value < 1:
                raise ValueError(f"{name} must be at least 1, not {value}")
        if max_prefills_per_step is not None and max_prefills_per_step < 1:
            raise ValueError(f"max_prefills_per_step must be at least 1, not {max_prefills_per_step}")
        self._executor = executor
        self._max_batch, self._budget, self._max_prefills = max_batch, max_tokens_per_step, max_prefills_per_step
        self._step_ahead = step_ahead and all(hasattr(executor, name) for name in ("launch", "collect"))
        self._in_flight: _Flight | None = None
        # Request, or a _Live that was preempted. deque.append / popleft / appendleft are atomic: another
        # thread may submit while this one steps.
        self._queue: collections.deque = collections.deque()
        self._live: list[_Live] = []
        self._ids = self._admissions = 0
        self._tally = _Tally()
        self._closed_with: str | None = None
        self._gate = threading.Lock()   # submit against shutdown; nothing else is shared between threads

    # --- the caller's side -----------------------------------------------------------------------
    def submit(self, request: Request) -> None:
        """May be called from another thread than the one that steps. A request either reaches the queue before
        ``shutdown`` drains it, or hears the shutdown's message: never neither."""
        with self._gate:
            closed = self._closed_with
            if closed is None:
                self._queue.append(request)
        if closed is not None:
            request.on_error(closed)

    def has_work(self) -> bool:
        return bool(self._live or self._queue or self._in_flight is not None)

    def run_until_idle(self) -> None:
        while self.step():
            pass

    def shutdown(self, message: str = "the engine is shutting down") -> None:
        """Every live and waiting request hears ``message`` as its error and gives its pages back; a
        step in flight is forgotten; what is submitted afterwards fails at once."""
        with self._gate:   # whoever submits now has either appended already or will see the message
            self._closed_with = message
            waiting = list(self._queue)
            self._queue.clear()
        self._abandon_live(message)
        for item in waiting:
            (item.request if isinstance(item, _Live) else item).on_error(message)

    def stats(self) -> dict:
        t = self._tally
        return {
            "decode_steps": t.decode_steps,
            "tokens": t.delivered,
            "prefills": t.first_tokens,
            "mean_batch_size": t.decode_rows / max(1, t.decode_steps),
            "running": len(self._live),
            "waiting": len(self._queue),
            "steps": t.steps,
            "tokens_per_step": t.step_tokens / max(1, t.steps),
            "preemptions": t.preemptions,
            "dropped_tokens": t.dropped,   # computed past an end token nobody had seen yet
        }

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
        except Exception as error:
            # the step function serves all live requests at once: none of them can go on
            log.exception("the step failed; every live request ends with its message")
            self._abandon_live(str(error))
            return True
        return bool(entries) or self.has_work()

    # --- planning ------------------------------------------------------------------------------
    def _drop_cancelled(self) -> None:
        for live in [r for r in self._live if r.request.cancelled]:
            self._executor.close(live.request_id)
            self._live.remove(live)
            live.finished = True   # a token of its that is still in flight is dropped

    def _portion_that_fits(self, live: _Live, plan: _PagePlan, most: int):
        """(n, pages): the largest portion n <= most whose pages can be had beside what is planned
        already, and those pages per group; n = 0 if not even one token fits."""
        n = most
        while n >= 1:
            need = self._executor.pages_needed(live.request_id, n)
            if plan.fits(need):
                return n, need
            # shrink to the end of the page before the last one the portion touches
            length = self._executor.length(live.request_id)
            page = self._executor.page_size
            n = min(n - 1, ((length + n - 1) // page) * page - length)
        return 0, None

    def _preempt(self, victim: _Live) -> None:
        """The victim gives everything back and waits at the front of the queue; what it has been
        fed so far becomes prompt again, so that it is recomputed and goes on where it was."""
        assert not victim.awaiting, "a victim's tokens are all known"
        self._executor.close(victim.request_id)
        self._live.remove(victim)
        victim.pending = victim.history + victim.pending
        victim.history = []
        self._tally.preemptions += 1
        self._queue.appendleft(victim)

    def _plan(self):
        entries, owners = [], []
        plan = _PagePlan(self._executor.free_pages())
        budget = self._budget
        preempted = False
        # Live requests first, in admission order: decodes bring one token, prompts a portion.
        # Requests are planned oldest first and preempted youngest first, so a victim never has
        # an entry in the plan yet.
        for live in sorted(self._live, key=lambda r: r.order):
            if live not in self._live:
                continue  # preempted while an older request was planned
            if budget < 1:
                break
            if self._ends_in_flight(live):
                continue
            most = min(self._to_feed(live), budget)
            n, need = self._portion_that_fits(live, plan, most)
            while n == 0:
                if self._in_flight is not None:
                    raise _SettleFirst()   # nothing has been changed so far
                victim = max(self._live, key=lambda r: r.order)
                preempted = True
                if victim is live:
                    if len(self._live) == 1:
                        # alone, with every other page free, and still no room
                        self._executor.close(live.request_id)
                        self._live.remove(live)
                        live.request.on_error(self.NO_ROOM)
                    else:
                        self._preempt(live)
                    break
                self._preempt(victim)
                plan.free = self._executor.free_pages()
                n, need = self._portion_that_fits(live, plan, most)
            if n == 0:
                continue
            self._add_entry(entries, owners, plan, live, n, need)
            budget -= n
        # Then admissions, in arrival order; the head of the queue is never overtaken. None in a
        # step that had to preempt: the preempted request would come straight back.
        admitted = 0
        while not preempted and budget >= 1 and len(self._live) < self._max_batch and self._queue:
            if self._max_prefills is not None and admitted >= self._max_prefills:
                break
            item = self._queue.popleft()
            live = self._admit(item, plan, bool(entries))
            if live is None:
                continue          # cancelled or failed: the next one gets its turn
            if live is False:
                self._queue.appendleft(item)
                break             # no room yet: wait for a live request to end
            n, need = self._portion_that_fits(live, plan, min(len(live.pending), budget))
            self._add_entry(entries, owners, plan, live, n, need)
            budget -= n
            admitted += 1
        return entries, owners

    @staticmethod
    def _to_feed(live: _Live) -> int:
        return 1 if live.awaiting else len(live.pending)

    def _ends_in_flight(self, live: _Live) -> bool:
        """The token being sampled in the step in flight is this request's last, whatever it is."""
        if not live.awaiting:
            return False
        request, limit = live.request, self._executor.max_positions()
        return ((limit is not None and live.prompt_len + live.launched >= limit)
                or (request.max_new_tokens is not None and live.launched >= request.max_new_tokens))

    def _add_entry(self, entries, owners, plan, live, n, need) -> None:
        if live.awaiting:
            entry = StepEntry(live.request_id, [0], [0], from_slot=True)
        else:
            completes = n == len(live.pending)
            entry = StepEntry(live.request_id, list(live.pending[:n]), [n - 1] if completes else [])
        entries.append(entry)
        owners.append(live)
        plan.take(need)

    def _admit(self, item, plan, others_planned: bool):
        """None: the request is gone (cancelled / failed). False: no room now. Else the _Live."""
        request = item.request if isinstance(item, _Live) else item
        if request.cancelled:
            return None
        if isinstance(item, _Live):
            live = item
        else:
            try:
                prompt = list(request.prompt)
                if not prompt:
                    raise ValueError("the prompt has no tokens")
                self._executor.check_prompt(prompt)
            except Exception as error:
                log.warning("a request was refused at admission: %s", error)
                request.on_error(str(error))   # nobody else is touched by a prompt that cannot run
                return None
            live = _Live(request, prompt)
        if not self._executor.can_open():
            return False
        request_id = self._ids
        self._executor.open(request_id)
        # Admitted only if its whole prompt has room beside what is planned: a request that could
        # take a first portion and then stall would only be preempted again.
        if not plan.fits(self._executor.pages_needed(request_id, len(live.pending))):
            self._executor.close(request_id)
            if not self._live and not others_planned:
                request.on_error(self.NO_ROOM)
                return None
            return False
        self._ids += 1
        live.request_id = request_id
        live.order = self._admissions
        self._admissions += 1
        self._live.append(live)
        return live

    # --- running and delivering ----------------------------------------------------------------
    def _launch(self, entries, owners) -> _Flight:
        sampled = [o for o, e in zip(owners, entries) if e.want]
        sampling = [o.request.sampling for o in sampled]
        steps = [o.launched for o in sampled]
        if self._step_ahead:
            handle = self._executor.launch(entries, sampling, steps)
        else:
            handle = self._executor.run(entries, sampling, steps)
        tally = self._tally
        tally.steps += 1
        tally.step_tokens += sum(len(e.tokens) for e in entries)
        decodes = sum(1 for o, e in zip(owners, entries) if o.launched > 0 and len(e.tokens) == 1)
        if decodes:
            tally.decode_steps += 1
            tally.decode_rows += decodes
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
                self._tally.dropped += 1
                continue
            token = int(token)
            self._tally.first_tokens += owner.generated == 0
            owner.generated += 1
            if owner.fed_ahead:            # the step launched after this one has been fed it already
                owner.history.append(token)
                owner.fed_ahead = False
            else:
                owner.awaiting = False
                owner.pending = [token]
            self._hand_over(owner, token)
        self._live = [r for r in self._live if not r.finished]

    def _ending(self, live: _Live, token: int):
        """The reason this token ends its request, or None. First match wins:
        end token, then positions used up, then the request's own limit."""
        request, positions = live.request, self._executor.max_positions()
        checks = (
            (STOP, request.eos_token_id is not None and token == request.eos_token_id),
            (CONTEXT, positions is not None and live.prompt_len + live.generated >= positions),
            (LENGTH, request.max_new_tokens is not None and live.generated >= request.max_new_tokens),
        )
        return next((reason for reason, holds in checks if holds), None)

    def _hand_over(self, live: _Live, token: int) -> None:
        """One token to its request; if it is the last one, the pages go back now."""
        ending = self._ending(live, token)
        self._tally.delivered += 1
        try:
            live.request.on_token(token, ending)
        except Exception:
            log.exception("on_token raised: this request alone is dropped")
            ending = ending or STOP
        if ending is not None:
            live.finished = True
            self._executor.close(live.request_id)

    def _abandon_live(self, message: str) -> None:
        """Every live request ends with ``message``; the step in flight is forgotten."""
        abandoned, self._live, self._in_flight = self._live, [], None
        for live in abandoned:
            live.finished = True
            try:
                self._executor.close(live.request_id)
            except Exception:
                log.exception("a request's pages could not be given back after the step failed")
            live.request.on_error(message)

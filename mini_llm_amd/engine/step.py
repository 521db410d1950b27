"""The step function: one batch of (request, its next tokens) through the model and the cache.

The reference has three entry points (whole-prompt prefill of one sequence, decode of one token,
batched decode: engine/include/gpt2_gpu.h:64-68,89-90,161-165). Here there is one: portions of
prompts beside single decoded tokens, cut anywhere, run as one batch from the cache, with logits
returned only at the wanted places. Like the reference's calls it checks everything before it
changes anything (engine/src/gpt2_gpu_batch.cu:67-88), and a request's stored length grows only
after the step has been launched (engine/src/gpt2_gpu.cu:364).

A step in which every request brings one token and wants its logits (a decode step) is
launch-bound, as the reference found (docs/kernels/007_fewer_launches.md): it is captured once
per batch-size bucket in a HIP graph and replayed; the batch's metadata lies in a fixed device
buffer per bucket that is overwritten before each replay. Steps with portions of prompts are
captured too, per shape of batch, once a shape has come many times: up to a few thousand tokens of a
small model the host needs longer to launch the kernels than the GPU to run them."""

from __future__ import annotations

import gc
import time
from array import array as _array
from collections import OrderedDict

import numpy as np

from ..cache import CacheManager, OutOfPages
from .batch import BatchStaging, DecodeBatchBuilder, FixedBuffer, StepBatch, StepEntry, build_step_batch

GRAPH_BUCKETS = (1, 2, 4, 8, 16, 32, 64, 128, 256)
# Steps with portions of prompts: a step of a few thousand tokens of a small model is over on the GPU before the host has
# launched its kernels one by one (a mixed step of 512 tokens through the 24 layers of the medium shape: 3.1 ms of
# launching for 1.1 ms of work), so a shape of batch that keeps coming is captured too. The shapes of a serving run with a
# mixed load change from step to step (captured as they are, each at its second coming, they were captured for nothing:
# 7.5k generated tokens a second against 28.6k without), so a batch is laid out in a padded shape (build_step_batch's
# ``pad``): the short portions' rows in steps of 16, the long portions' rows in steps of 64 and their requests in powers
# of two. A serving run then sees a dozen shapes, not hundreds. A capture costs about 45 ms (most of it making the graph
# ready to launch) and a replay saves a millisecond, so a capture pays after some fifty replays: a shape is captured at its
# PORTION_GRAPH_AFTER-th coming (a shape that has come so often will come again), and enough shapes are kept that a steady
# load does not push its own shapes out (the least recently used one goes first, and counts anew). Larger steps are bound
# by the GPU and would only hold their activations' memory.
PORTION_GRAPH_AFTER = 4
PORTION_GRAPH_MAX_TOKENS = 8192
PORTION_GRAPHS_KEPT = 32
PORTION_SHAPES_COUNTED = 4096
PORTION_SHORT_ROWS, PORTION_LONG_ROWS = 16, 64   # the rows of short and of long portions are padded to multiples of these


class StepError(ValueError):
    """The batch cannot be run; nothing has been changed."""


# A decode step of many requests is one kernel bound by memory (attention over the cache) among six that wait for trips
# to memory with most compute units idle. From so many requests on (0: never) the captured step runs groups of its
# requests side by side, as branches of the graph, so that one group's small kernels run under another's attention.
# Off by default: the branches do overlap on the device (128 rows: 0.98 against 1.06 ms a step), but launching a graph
# with branches costs the host 4 to 5 us a kernel (0.78 ms for the 170 kernels of two groups), which at 64 and at 256
# rows is more than the device needs for the step, and a host that also schedules has less to spare than that.
DECODE_LANES_FROM = 0
DECODE_LANE_ROWS = 64    # the most requests of a group (the kernels for few rows take up to 64)
TOKEN_RING_ROWS = 8   # steps whose chosen tokens stay readable on the host after they were launched


class ChosenTokens:
    """The tokens a step chose on the device: ``device`` (int32, one per wanted row, valid until the next step) and, on
    the host, a row of page-locked memory. The row is complete once ``event`` has passed or, where the step's last
    kernel writes the row itself, once the row's last entry shows the step's ``number`` (``tolist`` waits for either).
    A row is used again ``TOKEN_RING_ROWS`` steps later."""

    __slots__ = ("device", "_host", "_n", "_event", "_number", "_flags")
    WAIT_SECONDS = 30.0

    def __init__(self, device, host, n, event=None, number=None, flags=1):
        self.device, self._host, self._n, self._event, self._number, self._flags = device, host, n, event, number, flags

    def __len__(self):
        return self._n

    def tolist(self) -> list:
        if self._event is not None:
            self._event.synchronize()
        else:
            self._await_number()
        return self._host[: self._n].tolist()

    def _await_number(self) -> None:
        """Spins on the row's last entries (each written by the device behind a share of the tokens, with a fence between);
        gives the processor away between looks once the first few thousand have found nothing."""
        row, number = self._host, self._number
        looks, deadline = 0, None
        flags = row[-self._flags:]
        while (flags != number).any():
            looks += 1
            if looks > 2000:
                time.sleep(0)
                if deadline is None:
                    deadline = time.monotonic() + self.WAIT_SECONDS
                elif time.monotonic() > deadline:
                    raise RuntimeError(f"the tokens of step {number} have not arrived after {self.WAIT_SECONDS:.0f} s (the row shows step {int(row[-1])})")


class _Lanes:
    """Streams side by side, for a step whose requests run their layers in groups (Model._layers_in_lanes): the first
    group stays on the stream the step runs on, every other gets a stream of its own, which waits for that stream at
    the fork and is waited for at the join. Inside a capture this gives the graph branches that the device runs at
    the same time. All streams have the default priority."""

    def __init__(self, device, parts: int = 2):
        import torch

        self.parts = parts
        self._streams = [torch.cuda.Stream(device=device) for _ in range(parts - 1)]
        self._main = None

    def cuts(self, rows: int) -> list:
        """Where the rows are cut: equal groups, in whole sixteens while there are that many rows."""
        unit = 16 if rows >= 16 * self.parts else 1
        per = -(-rows // (self.parts * unit)) * unit
        return [(lo, min(rows, lo + per)) for lo in range(0, rows, per)]

    def fork(self) -> None:
        import torch

        self._main = torch.cuda.current_stream()
        for stream in self._streams:
            stream.wait_stream(self._main)

    def lane(self, index: int):
        import contextlib

        import torch

        return contextlib.nullcontext() if index == 0 else torch.cuda.stream(self._streams[index - 1])

    def join(self) -> None:
        for stream in self._streams:
            self._main.wait_stream(stream)


class _DecodeGraph:
    """One captured decode step for up to ``capacity`` requests. ``chooses``: the captured step ends with the greedy
    choice of its tokens (models.TokenChoice) and moves its batch on by one token on the device, so that the next step
    of the same requests, each taking its token from its last-token slot, is replayed without anything being copied to
    the device before it or from the device after it: the tokens arrive in a ring of rows in page-locked host memory.
    ``draws``: such a step draws its tokens as each row's sampling parameters say (temperature, top-p; they and the count
    of tokens a request has drawn lie in the same device buffer, and the count moves on with the batch)."""

    def __init__(self, runner: "ModelRunner", capacity: int, chooses: bool = False, reach: int | None = None, draws: bool = False):
        import torch

        self.runner, self.capacity, self.chooses, self.draws = runner, capacity, chooses, draws and chooses
        self.builder = DecodeBatchBuilder(runner.cache, capacity, draws=self.draws)
        self.buffer = torch.zeros(len(self.builder.flat), dtype=torch.int32, device=runner.device)
        self.static_batch = self.builder.batch(self.buffer, [], reach)
        self.graph = None
        self.logits = None
        # from so many rows on the requests go through the layers in two groups side by side
        self.lanes = _Lanes(runner.device, max(2, capacity // DECODE_LANE_ROWS)) if runner.lanes_from and capacity >= runner.lanes_from else None
        if chooses:
            from ..ops import kernels

            self.flags = kernels.choose_flags(capacity)
            self.ring = torch.full((TOKEN_RING_ROWS, capacity + self.flags), -1, dtype=torch.int32).pin_memory()
            self.ring_rows = self.ring.numpy()   # the same memory, for the host's reads
            self.ring_at = 0        # the ring row the next step writes and that step's number: the host's count of the
            self.number = 0         # device's cursor
            self.on_device = None   # per row (request's cache entry, its table_changes, its length) that the device's batch stands at
            self.uploads = 0

    def run(self, entries, sampling=None):
        runner = self.runner
        if self.chooses:
            return self._run_choosing(entries, sampling)
        runner.staging.upload(self.builder.fill(entries), into=self.buffer)
        batch = self.static_batch
        batch.request_ids = [e.request_id for e in entries]
        if self.graph is None:
            self.graph, self.logits = _capture(runner, batch, lanes=self.lanes)
        self.graph.replay()
        return batch, self.logits[: len(entries)]

    def _run_choosing(self, entries, sampling=None):
        import torch

        from ..models.base import DrawParameters, TokenChoice

        runner, cache = self.runner, self.runner.cache
        records = [cache.requests[e.request_id] for e in entries]
        stands = self.on_device
        if self.draws:
            if sampling is None or len(sampling[0]) != len(entries) or len(sampling[1]) != len(entries):
                raise ValueError("a step that draws its tokens needs each row's sampling parameters and count of tokens drawn")
            hows, counts = sampling
        else:
            hows = counts = [None] * len(entries)
        # The device has moved the last step's batch on by itself. It is this step's batch if the same requests come
        # again in the same rows, each with the token in its slot, and no block table has changed since (a request that
        # reaches a new page, or gives one back, has: then everything is brought from the host as ever).
        carried_on = (stands is not None and len(stands) == len(records) and all(e.from_slot for e in entries)
                      and all(r is at[0] and r.table_changes == at[1] and r.length == at[2] and (how is at[3] or how == at[3]) and count == at[4]
                              for r, at, how, count in zip(records, stands, hows, counts)))
        if not carried_on:
            flat = self.builder.fill(entries)
            if self.draws:
                self.builder.fill_draws(hows, counts)
            self.builder.cursor[:] = (self.ring_at, self.number, 0)
            runner.staging.upload(flat, into=self.buffer)
            self.uploads += 1
        batch = self.static_batch
        batch.request_ids = [e.request_id for e in entries]
        if self.graph is None:
            draws = DrawParameters(*self.builder.draw_views(self.buffer)) if self.draws else None
            choice = TokenChoice(cache.last_token, host_ring=self.ring, cursor=self.builder.cursor_view(self.buffer), advance=True, draws=draws)
            self.graph, self.logits = _capture(runner, batch, choice, self.lanes)
        self.graph.replay()
        chosen = ChosenTokens(self.logits[: len(entries)], self.ring_rows[self.ring_at], len(entries), number=self.number, flags=self.flags)
        self.ring_at = (self.ring_at + 1) % TOKEN_RING_ROWS
        self.number = (self.number + 1) & 0x3FFFFFFF
        self.on_device = [(r, r.table_changes, r.length + 1, how, None if count is None else count + 1) for r, how, count in zip(records, hows, counts)]
        return batch, chosen


def _capture(runner, batch, choice=None, lanes=None):
    """Runs the batch once eagerly (on a side stream, as capture needs), then captures the same. With ``choice`` the
    captured step ends with the choice of its tokens; the eager run then chooses into memory of its own and moves
    nothing on, so that the first replay finds everything as the eager run found it."""
    import torch

    warm, extra = {}, {}
    if lanes is not None:
        warm["lanes"] = extra["lanes"] = lanes
    if choice is not None:
        extra["choice"] = choice
        from dataclasses import replace

        warm["choice"] = replace(choice, token_slots=torch.empty_like(choice.token_slots), host_ring=None, cursor=None, advance=False)
    side = torch.cuda.Stream(device=runner.device)
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        runner.forward(batch, **warm)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize(runner.device)
    graph = torch.cuda.CUDAGraph()
    # No garbage collection while the stream is being captured: it may finalise whatever lies around in reference
    # cycles, another engine's captured graphs among them, and giving their memory back is not permitted during a
    # capture (the process aborts). Collected before instead, and switched back on behind the capture.
    gc.collect()
    collecting = gc.isenabled()
    gc.disable()
    try:
        with torch.cuda.graph(graph):
            logits = runner.forward(batch, **extra)
    finally:
        if collecting:
            gc.enable()
    return graph, logits


class _PortionGraph:
    """One captured step for batches of one padded shape (so many rows of short portions, rows of long portions and long
    requests: build_step_batch's ``pad``). Everything else about a batch (tokens, positions, pages, which rows are real
    and which are wanted) lies in the device buffer that the kernels read, and is overwritten before each replay."""

    def __init__(self, runner: "ModelRunner", pad):
        self.runner, self.pad = runner, pad
        self.buffer = FixedBuffer(runner.device)
        self.graph = None
        self.logits = None
        self.batch = None

    def run(self, entries):
        runner = self.runner
        batch = build_step_batch(entries, runner.cache, runner.staging, vocab_size=runner.model.vocab_size, device_buffer=self.buffer,
                                 short_portion=runner.model.short_portion(), fixed_reach=True, pad=self.pad)
        if self.graph is None:
            self.graph, self.logits = _capture(runner, batch)
            self.batch = batch
        else:  # the captured kernels read the first batch's views of the buffer, which now holds this batch
            captured = self.batch
            same = (captured.n_tokens, captured.n_requests, captured.n_logit_rows, captured.max_q_len, captured.short_requests,
                    captured.short_rows, captured.max_total_len) == (batch.n_tokens, batch.n_requests, batch.n_logit_rows,
                                                                      batch.max_q_len, batch.short_requests, batch.short_rows, batch.max_total_len)
            if not same:
                raise RuntimeError("a captured step was asked to run a batch of another shape")
        self.graph.replay()
        wanted = sum(len(e.want) for e in entries)
        return batch, self.logits[:wanted] if wanted else None   # (the shape's further logit rows are padding)


class ModelRunner:
    def __init__(self, model, cache: CacheManager, device, use_graphs: bool = True, portion_graph_after: int | None = None,
                 lanes_from: int | None = None):
        """``portion_graph_after``: the time a shape of batch with portions of prompts has to come to be captured (None: the
        default, PORTION_GRAPH_AFTER; 0: never). ``lanes_from``: captured decode steps for at least so many requests run
        their layers in two groups side by side (None: the default, DECODE_LANES_FROM; 0: never)."""
        self.lanes_from = DECODE_LANES_FROM if lanes_from is None else int(lanes_from)
        self.model, self.cache, self.device = model, cache, device
        self.staging = BatchStaging(device) if device is not None else None
        self.steps_run = 0
        self.graph_steps = 0
        self.last_batch: StepBatch | None = None
        self.use_graphs = bool(use_graphs and device is not None and cache.max_length is not None and model.all_graph_safe())
        self._graphs: dict = {}
        self._decode_reaches = [r for r in model.decode_reaches() if cache.max_length is not None and r < cache.max_length]
        self._portion_graphs: OrderedDict = OrderedDict()   # shape of batch -> _PortionGraph, least recently used first
        self._shapes_seen: dict = {}                         # shape of batch -> how often it has come
        self.portion_graph_after = PORTION_GRAPH_AFTER if portion_graph_after is None else int(portion_graph_after)
        self.portion_graph_steps = 0
        self._token_rows, self._token_turn = [], 0
        self._sampler = None
        self.portion_graphs_made = 0      # captures of steps with prompt portions, and those given up for a newer shape
        self.portion_graphs_dropped = 0

    def drop_graphs(self) -> None:
        """Gives the captured steps back now (they and the runner refer to each other, so otherwise they would lie around
        until the garbage collector finds them)."""
        for graph in list(self._graphs.values()) + list(self._portion_graphs.values()):
            graph.runner = None
        self._graphs.clear()
        self._portion_graphs.clear()

    @staticmethod
    def _check_tokens(entry, vocab: int) -> None:
        """Every token an integer inside the vocabulary: a long portion is looked at as one array, and
        token by token only to name the one that is wrong."""
        tokens = entry.tokens
        entry.checked_tokens = None   # whatever an earlier step left: the list may have changed since
        if len(tokens) > 16:
            array = None
            if isinstance(tokens, np.ndarray):
                array = tokens
            elif isinstance(tokens, list):
                try:   # a third faster than numpy's own conversion of a list; anything but integers that fit is left to the loop below
                    array = np.frombuffer(_array("i", tokens), dtype=np.int32)
                except (ValueError, TypeError, OverflowError):
                    array = None
            if array is not None and array.ndim == 1 and array.dtype.kind in "iu" and 0 <= int(array.min()) and int(array.max()) < vocab:
                entry.checked_tokens = array.astype(np.int32, copy=False)
                return
        for token in tokens:
            if not isinstance(token, (int,)) and not hasattr(token, "__index__"):
                raise StepError(f"request {entry.request_id!r}: token {token!r} is not an integer")
            if not 0 <= int(token) < vocab:
                raise StepError(f"request {entry.request_id!r}: token {token} is outside the vocabulary [0, {vocab})")

    def longest_sequence(self) -> int | None:
        """The longest sequence a request may reach: the model's position limit or the cache's, whichever is less."""
        limits = [n for n in (self.model.max_positions(), self.cache.max_length) if n is not None]
        return min(limits) if limits else None

    def validate(self, entries) -> None:
        if not entries:
            raise StepError("a step needs at least one entry")
        seen = set()
        vocab, limit = self.model.vocab_size, self.longest_sequence()
        for entry in entries:
            if entry.request_id in seen:
                raise StepError(f"request {entry.request_id!r} appears twice in one step")
            seen.add(entry.request_id)
            if not self.cache.has(entry.request_id):
                raise StepError(f"request {entry.request_id!r} is not open")
            n = len(entry.tokens)
            if n < 1:
                raise StepError(f"request {entry.request_id!r} brings no tokens")
            if entry.from_slot and n != 1:
                raise StepError(f"request {entry.request_id!r}: only a single token can come from the last-token slot")
            if entry.from_slot and not self.cache.has_sampled_token(entry.request_id):
                raise StepError(f"request {entry.request_id!r}: no token has been sampled into its last-token slot yet")
            if not entry.from_slot:
                self._check_tokens(entry, vocab)
            length = self.cache.length(entry.request_id)
            if limit is not None and length + n > limit:
                raise StepError(f"request {entry.request_id!r}: {length} + {n} tokens exceed the {limit} positions a sequence may have")
            for w in entry.want:
                if not 0 <= int(w) < n:
                    raise StepError(f"request {entry.request_id!r}: wanted place {w} is not among its {n} tokens")

    def forward(self, batch, resolve: bool = True, observer=None, choice=None, lanes=None):
        """Tokens that come from last-token slots are fetched on the device, then the model runs."""
        extra = {}
        if observer is not None:
            extra["observer"] = observer
        if choice is not None:
            extra["choice"] = choice
        if lanes is not None:
            extra["lanes"] = lanes
        return self.model.forward(batch, self.cache, resolve_tokens=resolve, **extra)

    def _graph_for(self, entries, choose: bool = False, draws: bool = False):
        if not self.use_graphs:
            return None
        if any(len(e.tokens) != 1 or list(e.want) != [0] for e in entries):
            return self._portion_graph_for(entries)   # its tokens, if asked for, are chosen from its logits behind the replay
        if len(entries) > GRAPH_BUCKETS[-1]:
            return None
        capacity = next(b for b in GRAPH_BUCKETS if b >= len(entries))
        # the range of sequence lengths the step falls in, where the model's kernels differ between ranges
        reach = self.cache.max_length
        if self._decode_reaches:
            longest = max(self.cache.length(e.request_id) for e in entries) + 1
            reach = next((r for r in self._decode_reaches if r >= longest), reach)
        key = (capacity, choose, reach) + ((True,) if choose and draws else ())
        if key not in self._graphs:
            self._graphs[key] = _DecodeGraph(self, capacity, chooses=choose, reach=reach, draws=draws)
        return self._graphs[key]

    def _portion_graph_for(self, entries):
        """The captured step for batches of this shape, once the shape has come often enough."""
        if self.portion_graph_after <= 0:
            return None
        short = self.model.short_portion()
        lengths = [len(e.tokens) for e in entries]
        n_tokens = sum(lengths)
        if n_tokens > PORTION_GRAPH_MAX_TOKENS:
            return None
        # the padded shape the batch falls in: rows of short portions, rows of long portions, long requests
        short_rows, long_rows = sum(n for n in lengths if n <= short), sum(n for n in lengths if n > short)
        long_requests = sum(1 for n in lengths if n > short)
        round_up = lambda n, step: -(-n // step) * step
        shape = (round_up(short_rows, PORTION_SHORT_ROWS), round_up(long_rows, PORTION_LONG_ROWS),
                 1 << (long_requests - 1).bit_length() if long_requests else 0)
        if sum(len(e.want) for e in entries) > shape[0] + shape[2]:
            return None   # more wanted places than the shape has logit rows (a trace that wants every place): run as it is
        graph = self._portion_graphs.get(shape)
        if graph is not None:
            self._portion_graphs.move_to_end(shape)
            return graph
        if len(self._shapes_seen) >= PORTION_SHAPES_COUNTED:
            self._shapes_seen.clear()
        self._shapes_seen[shape] = self._shapes_seen.get(shape, 0) + 1
        if self._shapes_seen[shape] < self.portion_graph_after:
            return None
        while len(self._portion_graphs) >= PORTION_GRAPHS_KEPT:
            # A shape that loses its graph starts counting again: with more hot shapes than graphs are kept, each would
            # otherwise be captured anew every time its turn comes (a capture costs some forty steps' time).
            evicted, _ = self._portion_graphs.popitem(last=False)
            self._shapes_seen[evicted] = 0
            self.portion_graphs_dropped += 1
        graph = self._portion_graphs[shape] = _PortionGraph(self, shape)
        self.portion_graphs_made += 1
        return graph

    def step(self, entries: list[StepEntry], observer=None, choose: bool = False, sampling=None):
        """Runs the entries as one batch. Returns float32 logits [wanted places, vocab] on the
        device (None if nothing is wanted), in the order of the entries and of each ``want``;
        they are valid until the next step. Raises StepError / OutOfPages before anything has
        changed. ``observer(name, rows)`` is shown the residual stream after the embedding and
        after each layer, the rows in the order of the entries and of their tokens (such a step
        is not replayed from a graph).

        ``choose``: the step also chooses the greedy token at every wanted place, on the device, leaves it in the
        request's last-token slot and returns ``ChosenTokens`` instead of logits (a decode step does all of it inside
        its captured graph, and is replayed without a copy to or from the device while the same requests go on).
        ``sampling`` (with ``choose``): (one SamplingParams per wanted place, the number of tokens its request has drawn
        before this one), in the order of the logits: the tokens are drawn as those say instead of greedily."""
        self.validate(entries)
        if sampling is not None:
            wanted = sum(len(e.want) for e in entries)
            if not choose or len(sampling[0]) != wanted or len(sampling[1]) != wanted:
                raise StepError("sampling goes with choose=True, one parameter set and one count per wanted place")
            if all(how.greedy for how in sampling[0]):
                sampling = None
        reserved = []
        try:
            for entry in entries:
                self.cache.reserve(entry.request_id, len(entry.tokens))
                reserved.append(entry.request_id)
        except OutOfPages:
            for request_id in reserved:
                self.cache.rollback(request_id)
            raise
        try:
            graph = self._graph_for(entries, choose, sampling is not None) if observer is None else None
            if graph is not None:
                batch, logits = graph.run(entries, sampling) if isinstance(graph, _DecodeGraph) else graph.run(entries)
                if isinstance(graph, _PortionGraph):
                    self.portion_graph_steps += 1
                else:
                    self.graph_steps += 1
            else:
                batch = build_step_batch(entries, self.cache, self.staging, vocab_size=self.model.vocab_size, short_portion=self.model.short_portion())
                in_given_order = None
                if observer is not None:
                    rows = batch.rows_in_order_of([e.request_id for e in entries])
                    in_given_order = lambda name, hidden: observer(name, hidden[rows])
                logits = self.forward(batch, resolve=any(e.from_slot for e in entries), observer=in_given_order)
            if choose and not isinstance(logits, ChosenTokens):
                logits = self._choose_from_logits(logits, batch, sampling)
        except Exception:
            for request_id in reserved:
                self.cache.rollback(request_id)
            raise
        for entry in entries:
            self.cache.commit(entry.request_id, len(entry.tokens))
            if choose and entry.want:
                self.cache.note_sampled(entry.request_id)
        self.steps_run += 1
        self.last_batch = batch
        return logits

    def _choose_from_logits(self, logits, batch, sampling=None):
        """The tokens of a step that was not captured with its choice: the sampler over the logits (its argmax, or a draw
        as ``sampling`` says), each token left in its request's last-token slot."""
        if logits is None:
            return None
        if sampling is None:
            from ..ops import kernels

            tokens = kernels.sample(logits, token_slots=self.cache.last_token, slot_of_row=batch.logit_slots)
        else:
            if self._sampler is None:
                from ..sampling import Sampler

                self._sampler = Sampler(self.staging)
            tokens = self._sampler.sample(logits, list(sampling[0]), list(sampling[1]), token_slots=self.cache.last_token, slot_of_row=batch.logit_slots)
        return self.tokens_to_host(tokens, logits.shape[0])

    def tokens_to_host(self, tokens, n: int) -> ChosenTokens:
        """Queues the copy of ``n`` chosen tokens into page-locked host memory; ``ChosenTokens.tolist`` waits for that
        copy alone, not for what is launched after it."""
        import torch

        if not self._token_rows or self._token_rows[0].shape[0] < n:
            self._token_rows = [torch.empty(max(n, 64), dtype=torch.int32, pin_memory=True) for _ in range(TOKEN_RING_ROWS)]
        row = self._token_rows[self._token_turn % TOKEN_RING_ROWS]
        self._token_turn += 1
        row[:n].copy_(tokens[:n], non_blocking=True)
        event = torch.cuda.Event()
        event.record()
        return ChosenTokens(tokens, row.numpy(), n, event=event)

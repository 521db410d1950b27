"""One step's batch: the tokens of several requests laid end to end, with everything the
kernels need to find each token's request, position, cache rows and pages.

The reference packs the control data of a batched decode into one struct and uploads it with a
single pinned copy (engine/src/gpt2_gpu_batch.cu:18-24,91-113). The same is done here for mixed
batches; pages are numbers, not pointers."""

from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np


@dataclass
class StepEntry:
    """A request's next tokens (a portion of its prompt, or one decoded token) and the places
    among them whose logits are wanted."""

    request_id: object
    tokens: list   # of integers, or a one-dimensional integer array
    want: list = field(default_factory=list)
    # The (single) token is the one the sampler left in the request's last-token slot on the
    # device in an earlier step; ``tokens`` then holds a placeholder the host never looks at.
    from_slot: bool = False
    # the tokens as an int32 array, left here by whoever has converted them already (the step
    # function, when it checks a long portion), so that the batch is not built from the list again
    checked_tokens: object = field(default=None, repr=False, compare=False)

    def token_array(self) -> np.ndarray:
        array = self.checked_tokens
        if array is None or len(array) != len(self.tokens):
            array = np.asarray(self.tokens, dtype=np.int32)
        return array


@dataclass
class GroupStepData:
    block_tables: object   # int32 [n_requests, max_blocks]: pages of each request of the batch
    slots: object          # int32 [n_tokens]: cache row each token's key/value is written to


# Portions up to so many tokens are laid out before the longer ones, whatever the order of the
# entries, so that a mixer can treat the two kinds apart (single decoded tokens over long
# contexts beside long portions want different kernels) by cutting the batch at one row. How many
# is the model's to say (Model.short_portion: what its mixers' kernels for short portions take);
# this is what a batch built without a model gets.
SHORT_PORTION = 8


@dataclass
class StepBatch:
    n_tokens: int
    n_requests: int
    n_logit_rows: int
    max_q_len: int          # the longest portion in the batch
    short_requests: int     # the first so many requests bring portions of at most SHORT_PORTION tokens,
    short_rows: int         # which are the first so many rows; the requests after them bring longer ones
    short_portion: int = field(default=SHORT_PORTION, kw_only=True)   # the length that cut was made at
    first_row: int = field(default=0, kw_only=True)   # a part of a step's batch (rows_of_requests): its first row's place in the whole
    max_total_len: int      # the longest sequence after this step
    tokens: object          # int32 [n_tokens]
    positions: object       # int32 [n_tokens]
    token_request: object   # int32 [n_tokens]: row of the block tables (index into the batch)
    q_starts: object        # int32 [n_requests + 1]: first row of each request's portion
    context_lens: object    # int32 [n_requests]: tokens stored before this step
    state_slots: object     # int32 [n_requests]
    logit_rows: object      # int32 [n_logit_rows]: rows whose logits are computed
    token_sources: object   # int32 [n_tokens]: last-token slot a row's token is taken from, -1 = as given
    logit_slots: object     # int32 [n_logit_rows]: state slot of the request each logit row belongs to
    groups: list            # GroupStepData per cache group
    request_ids: list = field(default_factory=list)
    host: dict = field(default_factory=dict)   # the same arrays as numpy, for parts that plan on the host

    def rows_of_requests(self, lo: int, hi: int) -> "StepBatch":
        """Requests lo..hi-1 of a batch in which every request brings one token (a decode step) as a batch of their own,
        over the same device memory: row r of it is row lo + r of this one. The block tables stay whole (a row's
        ``token_request`` still names its line there)."""
        if self.max_q_len != 1 or self.n_requests != self.n_tokens or not 0 <= lo < hi <= self.n_tokens:
            raise ValueError("only a batch of single tokens can be cut between requests")
        n = hi - lo
        cut = lambda t: t[lo:hi]
        return StepBatch(
            n_tokens=n, n_requests=n, n_logit_rows=n, max_q_len=1, short_requests=n, short_rows=n, short_portion=self.short_portion,
            max_total_len=self.max_total_len, tokens=cut(self.tokens), positions=cut(self.positions), token_request=cut(self.token_request),
            q_starts=self.q_starts[lo : hi + 1], context_lens=cut(self.context_lens), state_slots=cut(self.state_slots),
            logit_rows=cut(self.logit_rows), token_sources=cut(self.token_sources), logit_slots=cut(self.logit_slots),
            groups=[GroupStepData(block_tables=g.block_tables, slots=cut(g.slots)) for g in self.groups],
            request_ids=self.request_ids[lo:hi], host={}, first_row=self.first_row + lo,
        )

    def rows_in_order_of(self, request_ids) -> list:
        """The batch's rows, listed request by request in the given order of the requests (the
        batch itself may lay the requests out in another order)."""
        starts = self.host["q_starts"]
        place = {request_id: i for i, request_id in enumerate(self.request_ids)}
        rows = []
        for request_id in request_ids:
            i = place[request_id]
            rows.extend(range(int(starts[i]), int(starts[i + 1])))
        return rows


class BatchStaging:
    """Pinned host buffers, used in turn, and the device buffer the batch is copied into. A
    buffer is written again only after the copy out of it has finished."""

    def __init__(self, device, ring: int = 4):
        self.device, self.ring = device, ring
        self._host, self._events, self._device = [], [], []
        self._next = 0
        self._capacity = 0

    def _grow(self, n_ints: int) -> None:
        import torch

        torch.cuda.synchronize(self.device)
        self._capacity = max(1024, 1 << (n_ints - 1).bit_length())
        self._host = [torch.empty(self._capacity, dtype=torch.int32, pin_memory=True) for _ in range(self.ring)]
        self._device = [torch.empty(self._capacity, dtype=torch.int32, device=self.device) for _ in range(self.ring)]
        self._events = [None] * self.ring

    def upload(self, flat: np.ndarray, into=None):
        """flat: int32 numpy array -> device tensor holding it (valid until ``ring`` later
        uploads), or copied into the device tensor ``into`` if one is given."""
        import torch

        n = int(flat.shape[0])
        if n > self._capacity:
            self._grow(n)
        i = self._next
        self._next = (i + 1) % self.ring
        if self._events[i] is not None:
            self._events[i].synchronize()
        self._host[i][:n].numpy()[:] = flat
        target = self._device[i][:n] if into is None else into[:n]
        target.copy_(self._host[i][:n], non_blocking=True)
        event = torch.cuda.Event()
        event.record()
        self._events[i] = event
        return target


class FixedBuffer:
    """The device buffer that a captured step reads its batch from: made when the first batch is laid out into it,
    and of that length from then on (a graph is replayed only for batches whose layout has the same length)."""

    def __init__(self, device):
        self.device = device
        self.tensor = None

    def take(self, n_ints: int):
        import torch

        if self.tensor is None:
            self.tensor = torch.zeros(n_ints, dtype=torch.int32, device=self.device)
        if n_ints != len(self.tensor):
            raise ValueError(f"a batch of {n_ints} numbers does not fit the {len(self.tensor)} this buffer was made for")
        return self.tensor


def _aligned(n: int) -> int:
    return (n + 3) & ~3  # sections start on 16-byte boundaries


def build_step_batch(entries, cache, staging: BatchStaging | None, *, vocab_size: int, capacity: int | None = None,
                     device_buffer=None, short_portion: int = SHORT_PORTION, fixed_reach: bool = False, pad=None) -> StepBatch:
    """Lays out the batch on the host and uploads it in one copy. The entries have been checked
    and their pages reserved. With ``staging`` None the arrays stay numpy (host-only tests).

    ``capacity`` pads the batch to that many tokens and requests with rows that do nothing (token
    -1, request -1, slot -1), so that the layout depends on the capacity alone; ``device_buffer``
    then is the fixed device buffer the batch is copied into (a captured graph reads it); a
    ``FixedBuffer`` is made to the batch's length at its first use. ``fixed_reach`` names the longest
    sequence the cache can hold as the longest of this batch, as a padded batch does, so that nothing
    a kernel launch is sized by depends on how far the requests have come.

    ``pad`` = (short rows, long rows, long requests) lays a batch of portions out in a padded shape, so that batches
    of many shapes share one layout (and one captured graph): the short portions' rows padded to so many rows (and as
    many requests), behind them the long portions' rows and requests padded likewise, and as many logit rows as there
    are short rows and long requests. Padding rows belong to no request (token -1, request -1, slot -1); padding
    requests have a stored length of -1 and no pages, and no rows among the long ones (among the short ones the last of
    them spans the padding rows, none of which names it: a kernel that goes request by request passes a request with
    a negative length by); padding logit rows name row 0 and no slot.

    The requests are laid out short portions first (up to ``short_portion`` tokens); the logit rows
    keep the order of the entries as given."""
    n_requests = len(entries)
    given = entries
    layout = sorted(range(n_requests), key=lambda i: len(given[i].tokens) > short_portion)  # stable
    place = {i: at for at, i in enumerate(layout)}   # entry as given -> its place in the layout
    entries = [given[i] for i in layout]
    q_lens = [len(e.tokens) for e in entries]
    short_requests = sum(1 for q in q_lens if q <= short_portion)
    short_rows = sum(q for q in q_lens if q <= short_portion)
    n_tokens = sum(q_lens)
    records = [cache.requests[e.request_id] for e in entries]
    contexts = [r.length for r in records]
    n_groups = len(cache.groups)
    page_size = cache.page_size
    max_total = max(c + q for c, q in zip(contexts, q_lens))
    table_width = cache.max_blocks() or max(1, -(-max_total // page_size))
    cap_tokens = n_tokens if capacity is None else capacity
    cap_requests = n_requests if capacity is None else capacity
    n_logit_rows = sum(len(e.want) for e in entries)
    logit_length = n_logit_rows if capacity is None else max(n_logit_rows, cap_tokens)
    request_at = list(range(n_requests))       # where each request of the layout lies among the (padded) requests
    first_long_row = short_rows                # and where the long portions' rows begin
    if pad is not None:
        if capacity is not None:
            raise ValueError("a batch is padded to a capacity or to a shape of portions, not both")
        pad_short_rows, pad_long_rows, pad_long_requests = (int(n) for n in pad)
        if (short_rows > pad_short_rows or n_tokens - short_rows > pad_long_rows or n_requests - short_requests > pad_long_requests
                or n_logit_rows > pad_short_rows + pad_long_requests or (pad_short_rows > short_rows and pad_short_rows <= short_requests)):
            raise ValueError("the batch exceeds the shape it is laid out for")
        cap_tokens, cap_requests = pad_short_rows + pad_long_rows, pad_short_rows + pad_long_requests
        logit_length = pad_short_rows + pad_long_requests
        request_at = [i if i < short_requests else pad_short_rows + (i - short_requests) for i in range(n_requests)]
        first_long_row = pad_short_rows
    if n_tokens > cap_tokens or n_requests > cap_requests:
        raise ValueError("the batch exceeds the capacity it is laid out for")

    # One flat array, its sections starting on 16-byte boundaries, filled in place (no section is built apart and copied):
    # tokens, positions, token_request, q_starts, context_lens, state_slots, logit_rows, token_sources,
    # (block table, slots) per cache group, logit_slots.
    lengths = [cap_tokens, cap_tokens, cap_tokens, cap_requests + 1, cap_requests, cap_requests, logit_length, cap_tokens]
    for _ in range(n_groups):
        lengths += [cap_requests * table_width, cap_tokens]
    lengths.append(logit_length)
    offsets, total = [], 0
    for length in lengths:
        offsets.append(total)
        total += _aligned(length)
    flat = np.zeros(max(total, 4), dtype=np.int32)
    sections = [flat[o : o + n] for o, n in zip(offsets, lengths)]
    tokens, positions, token_request, q_starts, context_lens, state_slots, logit_rows, token_sources = sections[:8]

    starts, ends, at_row = [], [], 0
    for i, q in enumerate(q_lens):
        if i == short_requests:
            at_row = first_long_row
        starts.append(at_row)
        at_row += q
        ends.append(at_row)
    tokens[:] = -1
    token_request[:] = -1
    token_sources[:] = -1
    # a request's rows are q_starts[r] .. q_starts[r + 1]: a padding request begins where the request before it ends
    q_starts[:] = n_tokens if pad is None else (ends[-1] if n_requests > short_requests else first_long_row)
    if pad is not None:
        q_starts[short_requests : pad[0]] = short_rows
        context_lens[:] = -1   # a padding request: kernels that go request by request pass it by
    for i in range(n_requests):
        q_starts[request_at[i]] = starts[i]
        context_lens[request_at[i]] = contexts[i]
    if pad is None:
        q_starts[n_requests] = n_tokens
    state_slots[:] = -1    # padding: no request, no slot
    for i, e in enumerate(entries):
        lo, hi = starts[i], ends[i]
        tokens[lo:hi] = e.token_array()
        positions[lo:hi] = np.arange(contexts[i], contexts[i] + q_lens[i], dtype=np.int32)
        token_request[lo:hi] = request_at[i]
        state_slots[request_at[i]] = records[i].state_slot
        if e.from_slot:
            token_sources[lo] = records[i].state_slot
    tables, slots = [], []
    for gi in range(n_groups):
        table = sections[8 + 2 * gi].reshape(cap_requests, table_width)
        slot = sections[9 + 2 * gi]
        table[:] = -1
        slot[:] = -1
        for i, e in enumerate(entries):
            lo, hi = starts[i], ends[i]
            pages = np.asarray(cache.block_table(e.request_id, gi), dtype=np.int32)
            table[request_at[i], : len(pages)] = pages
            pos = positions[lo:hi]
            slot[lo:hi] = pages[pos // page_size] * page_size + pos % page_size
        tables.append(table)
        slots.append(slot)
    logit_slots = sections[-1]
    logit_slots[:] = -1
    at = 0
    for i, e in enumerate(given):
        for w in e.want:
            logit_rows[at] = starts[place[i]] + w
            logit_slots[at] = records[place[i]].state_slot
            at += 1

    host = {"tokens": tokens[:n_tokens], "positions": positions[:n_tokens], "token_request": token_request[:n_tokens],
            "q_starts": q_starts[: n_requests + 1], "context_lens": context_lens[:n_requests], "state_slots": state_slots[:n_requests],
            "logit_rows": logit_rows[:n_logit_rows], "token_sources": token_sources[:n_tokens], "logit_slots": logit_slots[:n_logit_rows],
            "block_tables": tables, "slots": slots}
    if staging is None:
        views = sections
    else:
        if isinstance(device_buffer, FixedBuffer):
            device_buffer = device_buffer.take(len(flat))
        device = staging.upload(flat, into=device_buffer)
        views = [device[o : o + n] for o, n in zip(offsets, lengths)]
    groups = [
        GroupStepData(block_tables=views[8 + 2 * gi].reshape(cap_requests, table_width), slots=views[9 + 2 * gi])
        for gi in range(n_groups)
    ]
    longest = max(q_lens)
    if pad is not None:   # what a launch is sized by depends on the shape alone
        short_requests = short_rows = pad[0]
        longest = pad[1] if pad[1] > 0 else short_portion
    return StepBatch(
        n_tokens=cap_tokens, n_requests=cap_requests, n_logit_rows=logit_length, max_q_len=longest,
        short_requests=short_requests, short_rows=short_rows,
        max_total_len=max_total if capacity is None and pad is None and not fixed_reach else (cache.max_length or table_width * page_size),
        tokens=views[0], positions=views[1], token_request=views[2], q_starts=views[3], context_lens=views[4],
        state_slots=views[5], logit_rows=views[6], token_sources=views[7], logit_slots=views[-1], groups=groups,
        request_ids=[e.request_id for e in entries], host=host, short_portion=short_portion,
    )


class DecodeBatchBuilder:
    """The same layout as ``build_step_batch(..., capacity=...)`` for the one case that runs every
    few hundred microseconds: every request brings one token and wants its logits. The padded
    arrays are kept and only the rows of the live requests are rewritten, so a step costs a short
    loop instead of a dozen array constructions."""

    def __init__(self, cache, capacity: int, draws: bool = False):
        """``draws``: the step also draws its tokens on the device (temperature, top-p): room for each row's seed,
        temperature, nucleus mass and count of tokens drawn so far."""
        self.cache, self.capacity = cache, capacity
        self.table_width = cache.max_blocks()
        n_groups = len(cache.groups)
        lengths = [capacity] * 3 + [capacity + 1] + [capacity] * 4
        for _ in range(n_groups):
            lengths += [capacity * self.table_width, capacity]
        lengths.append(3)   # for a step that chooses its tokens on the device: the row of the token ring it writes next, its number, and a count that is zero between steps
        if draws:
            lengths += [2 * capacity, capacity, capacity, capacity]   # seeds (64-bit), temperatures, nucleus masses (32-bit floats), counts
        self.offsets, total = [], 0
        for n in lengths:
            self.offsets.append(total)
            total += _aligned(n)
        self.lengths = lengths
        self.flat = np.zeros(max(total, 4), dtype=np.int32)
        view = lambda i: self.flat[self.offsets[i] : self.offsets[i] + lengths[i]]
        self.tokens, self.positions, self.token_request, self.q_starts = view(0), view(1), view(2), view(3)
        self.context_lens, self.state_slots, self.logit_rows, self.token_sources = view(4), view(5), view(6), view(7)
        self.tables = [view(8 + 2 * g).reshape(capacity, self.table_width) for g in range(n_groups)]
        self.slots = [view(9 + 2 * g) for g in range(n_groups)]
        self.cursor = view(8 + 2 * n_groups)
        self.draws = draws
        if draws:
            at = 9 + 2 * n_groups
            self.seeds, self.temperatures, self.top_ps = view(at).view(np.int64), view(at + 1).view(np.float32), view(at + 2).view(np.float32)
            self.draw_counts = view(at + 3)
        self.filled = capacity  # rows that held a request in the previous step (all, so the first fill pads all)

    def fill_draws(self, sampling, counts) -> None:
        """How each row draws its token (objects with temperature, top_p and seed; a temperature of 0 or less: greedily)
        and how many tokens its request has drawn so far. Padding rows draw greedily."""
        n = len(sampling)
        self.seeds[:n] = [p.seed & 0x7FFFFFFFFFFFFFFF for p in sampling]
        self.temperatures[:n] = [max(p.temperature, 0.0) for p in sampling]
        self.top_ps[:n] = [p.top_p for p in sampling]
        self.draw_counts[:n] = counts
        self.seeds[n:], self.temperatures[n:], self.top_ps[n:], self.draw_counts[n:] = 0, 0.0, 1.0, 0

    def draw_views(self, device_flat):
        """(seeds int64, temperatures, top_ps float32, counts int32) as views of the buffer on the device."""
        import torch

        at = 9 + 2 * len(self.tables)
        section = lambda i: device_flat[self.offsets[at + i] : self.offsets[at + i] + self.lengths[at + i]]
        return section(0).view(torch.int64), section(1).view(torch.float32), section(2).view(torch.float32), section(3)

    def fill(self, entries) -> np.ndarray:
        n, cache, page = len(entries), self.cache, self.cache.page_size
        stale = max(self.filled, n)
        self.tokens[:stale] = -1
        self.positions[:stale] = 0
        self.token_request[:stale] = -1
        self.q_starts[:] = n
        self.context_lens[:stale] = 0
        self.state_slots[:stale] = -1
        self.logit_rows[:] = 0
        self.token_sources[:stale] = -1
        for table, slots in zip(self.tables, self.slots):
            table[:stale] = -1
            slots[:stale] = -1
        for i, entry in enumerate(entries):
            request = cache.requests[entry.request_id]
            length = request.length
            self.tokens[i] = entry.tokens[0]
            self.positions[i] = length
            self.token_request[i] = i
            self.q_starts[i] = i
            self.context_lens[i] = length
            self.state_slots[i] = request.state_slot
            self.logit_rows[i] = i
            if entry.from_slot:
                self.token_sources[i] = request.state_slot
            for g, pages in enumerate(request.tables):
                self.tables[g][i, : len(pages)] = pages
                self.slots[g][i] = pages[length // page] * page + length % page
        self.filled = n
        return self.flat

    def batch(self, device_flat, entries, reach: int | None = None) -> StepBatch:
        """``reach``: the longest sequence, after the step, of any batch that will lie in these views (None: the
        cache's own limit)."""
        views = [device_flat[o : o + n] for o, n in zip(self.offsets, self.lengths)]
        n_groups = len(self.tables)
        groups = [GroupStepData(block_tables=views[8 + 2 * g].reshape(self.capacity, self.table_width), slots=views[9 + 2 * g])
                  for g in range(n_groups)]
        return StepBatch(
            n_tokens=self.capacity, n_requests=self.capacity, n_logit_rows=self.capacity, max_q_len=1,
            short_requests=self.capacity, short_rows=self.capacity,
            max_total_len=self.cache.max_length if reach is None else reach, tokens=views[0], positions=views[1], token_request=views[2],
            q_starts=views[3], context_lens=views[4], state_slots=views[5], logit_rows=views[6], token_sources=views[7],
            logit_slots=views[5],  # every request has one logit row, in its own place
            groups=groups, request_ids=[e.request_id for e in entries], host={},
        )

    def cursor_view(self, device_flat):
        at = self.offsets[8 + 2 * len(self.tables)]
        return device_flat[at : at + 3]

"""The cache manager: keys and values in pages with a block table per request and layer group,
and slots for per-request state of fixed size.

The reference gives each sequence one contiguous cache for the full context, pooled and reused
(engine/src/gpt2_gpu.cu:147-195, pytorch/src/mini_llm/native.py:327-364), and keeps its
fixed-size per-sequence state (the token queue) inside that object
(engine/include/gpt2_gpu_internal.h:38-56). Here memory is handed out page by page, groups of
layers with different needs have pools of their own, and what a request holds is given back
when it ends or when a window has passed it. Pages are not cleared: rows beyond a request's
length are never read (the reference's argument for its reset, engine/src/gpt2_gpu.cu:173-179)."""

from __future__ import annotations

from dataclasses import dataclass, field

from ..parts.base import LayerContext
from .pages import OutOfPages, PagePool, blocks_for, first_needed_block

NO_PAGE = -1


class CacheError(RuntimeError):
    pass


@dataclass
class RequestCache:
    request_id: object
    length: int = 0                                   # tokens whose keys and values are stored
    tables: list = field(default_factory=list)        # per group: page of each block (NO_PAGE once given back)
    state_slot: int = NO_PAGE
    reserved: int = 0                                 # tokens beyond ``length`` that have pages
    token_in_slot: bool = False                       # a sampler has left a token in the last-token slot since admission
    table_changes: int = 0                            # how often a block table of the request has changed (pages taken, given back)


class CacheManager:
    def __init__(self, groups, state_needs, *, num_pages, page_size: int, max_requests: int, dtype=None,
                 device=None, max_length: int | None = None):
        """groups: list of CacheGroupSpec; state_needs: {state layer: StateNeed}; num_pages: one
        number for every group or {group name: number}. ``device`` None keeps the bookkeeping only
        (tests of the manager's decisions need no GPU)."""
        if page_size < 1 or page_size & (page_size - 1):
            raise ValueError(f"page_size {page_size} is not a power of two")
        self.groups = list(groups)
        self.page_size, self.max_requests, self.max_length = page_size, max_requests, max_length
        counts = num_pages if isinstance(num_pages, dict) else {g.name: num_pages for g in self.groups}
        self.pools = [PagePool(counts[g.name]) for g in self.groups]
        self.group_of_layer = {layer: gi for gi, g in enumerate(self.groups) for layer in g.layers}
        self.requests: dict = {}
        self._free_slots = list(range(max_requests - 1, -1, -1))
        self.state_needs = dict(state_needs)
        self.device, self.dtype = device, dtype
        self.k_pages, self.v_pages, self.state = {}, {}, {}
        # Per request, whatever the model: the token the sampler chose last, kept on the device so
        # that the next step can start before the host has seen it (the reference keeps such a
        # token queue inside each cache object: engine/include/gpt2_gpu_internal.h:38-48).
        self.last_token = None
        if device is not None:
            import torch

            self.last_token = torch.zeros((max_requests,), dtype=torch.int32, device=device)

            for gi, g in enumerate(self.groups):
                shape = (len(g.layers), 2, self.pools[gi].num_pages, g.n_kv_heads, page_size, g.head_size)
                store = torch.empty(shape, dtype=dtype, device=device)
                for li, layer in enumerate(g.layers):
                    self.k_pages[layer], self.v_pages[layer] = store[li, 0], store[li, 1]
            for layer, need in self.state_needs.items():
                self.state[layer] = torch.zeros((max_requests, *need.shape), dtype=need.dtype, device=device)

    # -- requests ----------------------------------------------------------------------------------
    def has(self, request_id) -> bool:
        return request_id in self.requests

    def can_open(self) -> bool:
        return bool(self._free_slots)

    def open(self, request_id) -> RequestCache:
        """Admits a request: an empty block table per group and a state slot, zeroed."""
        if request_id in self.requests:
            raise CacheError(f"request {request_id!r} is already open")
        if not self._free_slots:
            raise OutOfPages(f"all {self.max_requests} request slots are taken")
        slot = self._free_slots.pop()
        for tensor in self.state.values():
            tensor[slot].zero_()
        entry = RequestCache(request_id, tables=[[] for _ in self.groups], state_slot=slot)
        self.requests[request_id] = entry
        return entry

    def close(self, request_id) -> None:
        """Gives back everything the request holds."""
        entry = self.requests.pop(request_id, None)
        if entry is None:
            raise CacheError(f"request {request_id!r} is not open")
        for pool, table in zip(self.pools, entry.tables):
            pool.give([p for p in table if p != NO_PAGE])
        self._free_slots.append(entry.state_slot)

    def length(self, request_id) -> int:
        return self._entry(request_id).length

    def note_sampled(self, request_id) -> None:
        """A sampler has been launched that leaves this request's token in its last-token slot."""
        self._entry(request_id).token_in_slot = True

    def has_sampled_token(self, request_id) -> bool:
        """Whether the request's last-token slot holds a token of its own (a slot keeps what its
        previous owner left until the new owner is sampled for the first time)."""
        return self._entry(request_id).token_in_slot

    def _entry(self, request_id) -> RequestCache:
        try:
            return self.requests[request_id]
        except KeyError:
            raise CacheError(f"request {request_id!r} is not open") from None

    # -- pages ---------------------------------------------------------------------------------------
    def pages_needed(self, request_id, n_new: int) -> list[int]:
        """Per group: pages that ``reserve(request_id, n_new)`` would take."""
        entry = self._entry(request_id)
        target = blocks_for(entry.length + n_new, self.page_size)
        return [max(0, target - len(table)) for table in entry.tables]

    def free_pages(self) -> list[int]:
        return [pool.num_free for pool in self.pools]

    def can_reserve(self, wanted) -> bool:
        """wanted: [(request_id, n_new)]. True if all of them fit at once."""
        need = [0] * len(self.groups)
        for request_id, n_new in wanted:
            for gi, n in enumerate(self.pages_needed(request_id, n_new)):
                need[gi] += n
        return all(n <= pool.num_free for n, pool in zip(need, self.pools))

    def reserve(self, request_id, n_new: int) -> None:
        """Pages for the next ``n_new`` tokens of the request, in every group, or OutOfPages with
        nothing taken."""
        entry = self._entry(request_id)
        if n_new < 1:
            raise CacheError("a step brings at least one token per request")
        if self.max_length is not None and entry.length + n_new > self.max_length:
            raise CacheError(f"request {request_id!r}: {entry.length} + {n_new} tokens exceed the longest sequence {self.max_length}")
        need = self.pages_needed(request_id, n_new)
        for gi, (n, pool) in enumerate(zip(need, self.pools)):
            if n > pool.num_free:
                raise OutOfPages(f"request {request_id!r} needs {n} pages of group {self.groups[gi].name}, {pool.num_free} are free")
        for table, n, pool in zip(entry.tables, need, self.pools):
            table.extend(pool.take(n))
        entry.table_changes += any(need)
        entry.reserved = max(entry.reserved, n_new)

    def commit(self, request_id, n_new: int) -> None:
        """The step has stored ``n_new`` tokens: the length grows, and pages that a window has
        passed (no later query can read them) go back to their pool."""
        entry = self._entry(request_id)
        if n_new > entry.reserved:
            raise CacheError(f"request {request_id!r} commits {n_new} tokens but reserved {entry.reserved}")
        entry.length += n_new
        entry.reserved = 0
        for group, pool, table in zip(self.groups, self.pools, entry.tables):
            if group.window is None:
                continue
            keep_from = first_needed_block(entry.length, group.window, self.page_size)
            passed = [b for b in range(min(keep_from, len(table))) if table[b] != NO_PAGE]
            pool.give([table[b] for b in passed])
            for b in passed:
                table[b] = NO_PAGE
            entry.table_changes += bool(passed)

    def rollback(self, request_id) -> None:
        """Undoes a reserve whose step did not run: pages beyond the stored length go back."""
        entry = self._entry(request_id)
        keep = blocks_for(entry.length, self.page_size)
        for pool, table in zip(self.pools, entry.tables):
            pool.give([p for p in table[keep:] if p != NO_PAGE])
            entry.table_changes += len(table) > keep
            del table[keep:]
        entry.reserved = 0

    def block_table(self, request_id, group_index: int) -> list[int]:
        return self._entry(request_id).tables[group_index]

    def slot(self, request_id, group_index: int, position: int) -> int:
        """The cache row of a position: page * page_size + offset."""
        page = self._entry(request_id).tables[group_index][position // self.page_size]
        if page == NO_PAGE:
            raise CacheError(f"position {position} of request {request_id!r} lies on a page that was given back")
        return page * self.page_size + position % self.page_size

    def max_blocks(self, group_index: int = 0) -> int | None:
        return None if self.max_length is None else blocks_for(self.max_length, self.page_size)

    # -- for the step function -----------------------------------------------------------------------
    def layer_context(self, batch, call) -> LayerContext:
        gi = self.group_of_layer.get(call.cache)
        return LayerContext(
            batch=batch,
            k_pages=self.k_pages.get(call.cache),
            v_pages=self.v_pages.get(call.cache),
            group=None if gi is None else batch.groups[gi],
            write_cache=call.write_cache,
            state=self.state.get(call.cache),
        )

    def read_kv(self, request_id, layer: int, rows: int):
        """The first ``rows`` keys and values of a request in one cache layer, gathered through
        its block table: ([rows, n_kv_heads, head_size], same). For tests and debugging (the
        reference's gpt2_gpu_kv_cache_copy_layer, engine/src/gpt2_gpu.cu:185-195)."""
        import torch

        gi = self.group_of_layer[layer]
        slots = torch.tensor([self.slot(request_id, gi, p) for p in range(rows)], device=self.device)
        pages, offsets = slots // self.page_size, slots % self.page_size
        return self.k_pages[layer][pages, :, offsets, :], self.v_pages[layer][pages, :, offsets, :]

    # -- invariants (tests call this after every operation) -----------------------------------------
    def check_invariants(self) -> None:
        for gi, pool in enumerate(self.pools):
            seen: dict = {}
            for entry in self.requests.values():
                for page in entry.tables[gi]:
                    if page == NO_PAGE:
                        continue
                    if page in seen:
                        raise AssertionError(f"page {page} of group {gi} is held by {seen[page]!r} and {entry.request_id!r}")
                    seen[page] = entry.request_id
            if set(seen) != pool.held_pages():
                raise AssertionError(f"group {gi}: tables hold {sorted(seen)}, the pool says {sorted(pool.held_pages())}")
            if len(seen) + pool.num_free != pool.num_pages:
                raise AssertionError(f"group {gi}: {len(seen)} held + {pool.num_free} free != {pool.num_pages}")
        slots = [e.state_slot for e in self.requests.values()]
        if len(set(slots)) != len(slots) or set(slots) & set(self._free_slots):
            raise AssertionError("a state slot is held twice or is both held and free")
        if len(slots) + len(self._free_slots) != self.max_requests:
            raise AssertionError("a state slot was lost")
        for entry in self.requests.values():
            for group, table in zip(self.groups, entry.tables):
                if len(table) < blocks_for(entry.length, self.page_size):
                    raise AssertionError(f"request {entry.request_id!r}: table shorter than its length")
                first = first_needed_block(entry.length, group.window, self.page_size)
                if any(p == NO_PAGE for p in table[first:]):
                    raise AssertionError(f"request {entry.request_id!r}: a page inside the window is missing")

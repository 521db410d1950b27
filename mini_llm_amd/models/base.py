"""A model as data: parts, distinct layers, and the order in which layers run.

``schedule`` is a list of layer calls. A call names the layer (block) to run and the cache
layer it uses; the same block may be called twice (shared weights, a cache of its own each
time), and a call may read a cache layer that an earlier call wrote (``write_cache=False``)."""

from __future__ import annotations

from dataclasses import dataclass

from ..ops import kernels
from ..parts.base import Norm, Part, PositionEncoding
from ..parts.embedding import TokenEmbedding


@dataclass(frozen=True)
class LayerCall:
    block: int               # index into Model.blocks
    cache: int               # cache layer (and state layer) this call uses
    write_cache: bool = True


@dataclass(frozen=True)
class CacheGroupSpec:
    """Cache layers with the same page geometry and the same retention share one pool of page
    numbers and one block table per request."""

    name: str
    layers: tuple            # cache layer ids
    n_kv_heads: int
    head_size: int
    window: int | None


@dataclass
class DrawParameters:
    """How the rows of a step draw their tokens, one entry a wanted row, on the device: ``seeds`` (int64),
    ``temperatures`` (float32; 0: the argmax), ``top_ps`` (float32) and ``counts`` (int32: the tokens the row's request
    has drawn so far; the random numbers are a function of seed and count, kernels.sample)."""

    seeds: object
    temperatures: object
    top_ps: object
    counts: object


@dataclass
class TokenChoice:
    """Asks a step to choose its tokens on the device as its last kernel: one token per wanted row, the greedy one
    or, with ``draws``, one drawn as those say; left in the request's last-token slot (``token_slots``: the cache's), and,
    with ``host_ring`` / ``cursor``, in a ring of rows in page-locked host memory (kernels.choose). ``advance``: a step of
    single tokens also moves its batch on by one token on the device (and the counts of ``draws``), so that the same
    requests' next step needs nothing from the host."""

    token_slots: object
    host_ring: object = None
    cursor: object = None
    advance: bool = False
    draws: DrawParameters | None = None


class Model(Part):
    def __init__(self, config, precision, *, embedding: TokenEmbedding, position_encoding: PositionEncoding | None,
                 blocks: list, schedule: list, final_norm: Norm, head, names: dict):
        self.config, self.precision = config, precision
        self.embedding, self.position_encoding = embedding, position_encoding
        self.blocks, self.schedule = list(blocks), list(schedule)
        self.final_norm, self.head = final_norm, head
        self._names = names  # prefixes: embedding, position_encoding, block (format with {i}), final_norm
        written = set()
        for call in self.schedule:
            if not 0 <= call.block < len(self.blocks):
                raise ValueError(f"the schedule names layer {call.block}, but there are {len(self.blocks)}")
            if call.write_cache:
                if call.cache in written:
                    raise ValueError(f"cache layer {call.cache} is written by two layer calls")
                written.add(call.cache)
            elif call.cache not in written:
                raise ValueError(f"a layer call reads cache layer {call.cache} before any call has written it")

    # -- tree ------------------------------------------------------------------------------------
    def children(self):
        out = {self._names["embedding"]: self.embedding}
        if self.position_encoding is not None:
            out[self._names["position_encoding"]] = self.position_encoding
        for i, block in enumerate(self.blocks):
            out[self._names["block"].format(i=i)] = block
        out[self._names["final_norm"]] = self.final_norm
        return out

    def canonical_tensor_name(self, name: str) -> str | None:
        """Name in a file -> name in ``named_tensor_specs`` (None: known and not needed)."""
        return name

    # -- what the engine asks ----------------------------------------------------------------------
    @property
    def vocab_size(self) -> int:
        return self.embedding.vocab_size

    def max_positions(self) -> int | None:
        """The longest sequence the model can hold (None: no limit of its own)."""
        if self.position_encoding is not None and hasattr(self.position_encoding, "max_positions"):
            return self.position_encoding.max_positions()
        return None

    def short_portion(self) -> int:
        """The longest portion that the batch lays out among the short ones: what every mixer's
        kernel for short portions takes (a mixer without such a kernel does not care)."""
        limits = [limit for limit in (block.mixer_part().short_portion for block in self.blocks) if limit is not None]
        return min(limits) if limits else 1

    def decode_reaches(self) -> list[int]:
        """The sequence lengths at which some mixer decodes through other kernels, ascending: the engine keeps a
        captured decode step for each range between them."""
        return sorted({int(reach) for block in self.blocks for reach in block.mixer_part().decode_reaches})

    def cache_groups(self) -> list[CacheGroupSpec]:
        groups: dict = {}
        for call in self.schedule:
            need = self.blocks[call.block].mixer_part().kv_need()
            if need is None:
                continue
            layers = groups.setdefault((need.n_kv_heads, need.head_size, need.window), [])
            if call.write_cache:
                layers.append(call.cache)
            elif call.cache not in layers:
                raise ValueError(f"a layer call reads cache layer {call.cache}, whose pages have another shape or window")
        return [
            CacheGroupSpec(f"{'window' + str(key[2]) if key[2] else 'full'}_h{key[0]}x{key[1]}", tuple(layers), *key)
            for key, layers in groups.items()
        ]

    def state_needs(self) -> dict:
        """state layer id -> StateNeed, for the mixers that keep state of fixed size."""
        out = {}
        for call in self.schedule:
            need = self.blocks[call.block].mixer_part().state_need()
            if need is not None and call.write_cache:
                out[call.cache] = need
        return out

    def _layers(self, hidden, batch, cache, observer=None):
        """The schedule over the rows of ``batch``; the stream comes back as the last layer leaves it."""
        for index, call in enumerate(self.schedule):
            block = self.blocks[call.block]
            if not block.takes_pending:
                hidden = kernels.settle(hidden)
            hidden = block.forward(hidden, cache.layer_context(batch, call))
            if observer is not None:
                observer(index, kernels.settle(hidden))
        return hidden

    def _layers_in_lanes(self, hidden, batch, cache, lanes):
        """A decode step's requests in ``lanes.parts`` groups of neighbouring rows, each group through all layers and the
        final norm on a lane (a stream) of its own: nothing in a layer connects two requests, and while one group's
        attention reads its keys and values (bound by memory) the other's products, which wait for one trip to memory
        after the other, find the compute units free. Returns the normalised rows of all groups, [rows, width], for the
        head, which reads its matrix once for all of them."""
        import torch

        rows = batch.n_tokens
        normed = torch.empty((rows, hidden.shape[1]), dtype=self.precision.compute, device=hidden.device)
        hidden = kernels.settle(hidden)
        cuts = lanes.cuts(rows)
        lanes.fork()
        kept = []   # what one lane made stays alive until all have joined: its memory must not go to another lane meanwhile
        for lane, (lo, hi) in enumerate(cuts):
            with lanes.lane(lane):
                part = batch.rows_of_requests(lo, hi)
                out = self._layers(hidden[lo:hi], part, cache)
                if not self.final_norm.takes_pending:
                    out = kernels.settle(out)
                self.final_norm.forward_into(out, normed[lo:hi])
                kept.append((part, out))
        lanes.join()
        del kept
        return normed

    def forward(self, batch, cache, resolve_tokens: bool = False, observer=None, choice: TokenChoice | None = None, lanes=None):
        """The whole step: embeds the batch's tokens, runs the schedule over the cache, and
        returns float32 logits [len(batch.logit_rows), vocab] at the wanted rows only (with
        ``choice``: the greedy token of each wanted row instead, int32 on the device). With
        ``resolve_tokens`` the rows that name a last-token slot take their token from it.
        ``lanes`` (fork(), lane(i), join(), cuts(rows)): a step of single tokens runs its layers in groups of requests
        side by side (``_layers_in_lanes``).
        ``observer(name, rows)``, if given, is shown the residual stream (float32 [tokens, width],
        rows in the batch's order) after the embedding (name "embedding") and after each entry of
        the schedule (its index): what the reference's block_outputs are for, finding the layer
        where a difference starts (engine/include/gpt2_gpu.h:21-25). The step itself runs as without."""
        hidden = self.embedding.forward(batch.tokens, batch.positions, self.position_encoding,
                                        token_sources=batch.token_sources if resolve_tokens else None,
                                        token_slots=cache.last_token if resolve_tokens else None)
        if observer is not None:
            observer("embedding", kernels.settle(hidden))
        if lanes is not None:
            normed = self._layers_in_lanes(hidden, batch, cache, lanes)
        else:
            hidden = self._layers(hidden, batch, cache, observer)
            if batch.n_logit_rows == 0:
                return None
            if not self.final_norm.takes_pending:
                hidden = kernels.settle(hidden)
            # the final norm runs on the wanted rows only (engine/src/gpt2_gpu.cu:254-258)
            normed = self.final_norm.forward(hidden, self.precision.compute, row_index=batch.logit_rows)
        if choice is None:
            return self.head.forward(normed)
        # Greedy tokens on the device. A head that can leave the best of its columns instead of all of them does (the
        # logits of a greedy step are read by nobody); any other head's logits go through the sampler's argmax.
        draws = choice.draws
        best = self.head.forward_best(normed) if draws is None and hasattr(self.head, "forward_best") else None
        if draws is not None:    # drawn from the logits; what is left to choose from is the one token a row
            values, indices = None, kernels.sample(self.head.forward(normed), draws.temperatures, draws.top_ps, draws.seeds, draws.counts).view(-1, 1)
        elif best is None:
            values, indices = None, kernels.sample(self.head.forward(normed)).view(-1, 1)
        else:
            values, indices = best
        advance = None
        if choice.advance:
            if batch.max_q_len != 1 or batch.n_logit_rows != batch.n_tokens:
                raise ValueError("only a step of single tokens that all want their logits can be moved on by one on the device")
            advance = kernels.StepAdvance(batch.positions, batch.context_lens, batch.token_sources, [g.block_tables for g in batch.groups],
                                          [g.slots for g in batch.groups], cache.page_size,
                                          draw_counts=None if draws is None else draws.counts)
        return kernels.choose(values, indices, batch.logit_slots, choice.token_slots, host_ring=choice.host_ring, cursor=choice.cursor,
                              advance=advance)

"""The interfaces of the parts a layer is put together from, and one registry per kind.

A part owns its sizes and constants as constructor parameters, declares the tensors it needs
(``tensor_specs``), receives them (``bind``) and computes (``forward``). No part knows which
model it is in: the architecture's builder picks parts by name, layer by layer."""

from __future__ import annotations

from dataclasses import dataclass, field

from ..weights.spec import TensorSpec


class Part:
    """A node of the model tree: its own tensors plus named children."""

    # True if ``forward`` only launches kernels whose arguments are device tensors and numbers
    # fixed by the batch's capacity: then a decode step may be captured in a HIP graph and
    # replayed. A part that plans on the host from the batch's contents says False.
    graph_safe = True

    def tensor_specs(self) -> dict[str, TensorSpec]:
        """local tensor name -> spec, for this part's own tensors."""
        return {}

    def children(self) -> dict[str, "Part"]:
        """name prefix -> sub-part."""
        return {}

    def bind(self, tensors: dict) -> None:
        """Receives this part's own tensors, already on the device in the kept layout."""
        for name, tensor in tensors.items():
            setattr(self, name.replace(".", "_"), tensor)

    # -- walking the tree ------------------------------------------------------------------
    def named_tensor_specs(self, prefix: str = "") -> dict[str, TensorSpec]:
        out = {prefix + name: spec for name, spec in self.tensor_specs().items()}
        for child_prefix, child in self.children().items():
            out.update(child.named_tensor_specs(prefix + child_prefix))
        return out

    def all_graph_safe(self) -> bool:
        return self.graph_safe and all(child.all_graph_safe() for child in self.children().values())

    def bind_named(self, tensors: dict, prefix: str = "") -> None:
        own = {name: tensors[prefix + name] for name in self.tensor_specs()}
        if own:
            self.bind(own)
        for child_prefix, child in self.children().items():
            child.bind_named(tensors, prefix + child_prefix)


# -- what a mixer may ask of the cache manager ---------------------------------------------------
@dataclass(frozen=True)
class KVNeed:
    """Keys and values that grow with the sequence, kept in pages. ``window`` None: every key
    is kept; an integer w: only the last w keys are ever read, older pages are given back."""

    n_kv_heads: int
    head_size: int
    window: int | None = None


@dataclass(frozen=True)
class StateNeed:
    """State of fixed size per request, kept in a slot: zero at admission, updated in place."""

    shape: tuple
    dtype: object  # torch.dtype


@dataclass
class LayerContext:
    """What the step function hands a mixer for one layer call."""

    batch: object                 # engine.batch.StepBatch: tokens, positions, requests
    k_pages: object = None        # [num_pages, n_kv_heads, page_size, head_size] of the call's cache layer
    v_pages: object = None
    group: object = None          # cache.GroupStepData: block tables and write slots of the layer's group
    write_cache: bool = True      # False: the layer reads a cache another layer call has written
    state: object = None          # [num_slots, *StateNeed.shape] of the call's state layer
    extra: dict = field(default_factory=dict)


class Norm(Part):
    # True if ``forward`` also takes rows whose last sums are pending (ops.kernels.PendingRows)
    takes_pending = False

    def forward(self, x, out_dtype, row_index=None):
        """x: [rows, width] float32 -> [rows or len(row_index), width] of out_dtype."""
        raise NotImplementedError

    def forward_into(self, x, out):
        """The normalised rows of x written into ``out`` ([rows, width], its element type the one asked for): for a
        caller that gathers the rows of several calls in one tensor. A norm whose kernel can write where it is told
        overrides this; the default copies."""
        from ..ops import kernels

        return kernels.convert(self.forward(x, out.dtype), out.dtype, out=out)

    def forward_with_sums(self, hidden, out_dtype, packed=False):
        """hidden: float32 rows, or rows whose last sums are pending -> (the normalised rows, the
        rows with their sums taken: what the residual stream goes on with). A norm that can take
        the sums on its way in overrides this. ``packed``: the caller would like the normalised
        rows as kernels.PackedRows (it takes plain rows too: this default gives those)."""
        from ..ops import kernels

        hidden = kernels.settle(hidden)
        return self.forward(hidden, out_dtype), hidden


class Mixer(Part):
    """Mixes information between the positions of a sequence (attention here)."""

    graph_safe = False  # a mixer says so itself
    # Portions up to so many tokens this mixer runs through a kernel of their own, apart from longer
    # ones (None: it makes no difference): the batch lays such portions out first.
    short_portion: int | None = None
    # Sequence lengths at which this mixer's kernels for decoding change: a captured decode step is made for each range
    # between them, and learns the range's end as the longest sequence of its batch (StepBatch.max_total_len).
    decode_reaches: tuple = ()

    def kv_need(self) -> KVNeed | None:
        return None

    def state_need(self) -> StateNeed | None:
        return None

    def forward(self, x, residual, ctx: LayerContext):
        """x: [rows, width] normed input in the compute dtype; returns residual + mix(x) in
        float32 (plain rows, or rows whose last sums are pending: ops.kernels.PendingRows). Rows belong to several requests and may be a portion of a prompt or one decoded
        token; what came before is in the cache / the state slot."""
        raise NotImplementedError

    def forward_normed(self, hidden, norm: Norm, compute_dtype, ctx: LayerContext):
        """norm, then ``forward``, then the residual sum, as one call: a mixer that has a kernel
        for the whole chain overrides this. ``hidden`` and the result are float32 rows or rows
        whose last sums are pending (ops.kernels.PendingRows)."""
        x, hidden = norm.forward_with_sums(hidden, compute_dtype)
        return self.forward(x, hidden, ctx)


class FeedForward(Part):
    def forward(self, x, residual):
        """x: [rows, width] in the compute dtype; returns residual + f(x) in float32 (plain rows, or
        rows whose last sums are pending)."""
        raise NotImplementedError

    def forward_normed(self, hidden, norm: Norm, compute_dtype, ctx: LayerContext):
        """norm, then ``forward``, then the residual sum, as one call (see Mixer.forward_normed)."""
        x, hidden = norm.forward_with_sums(hidden, compute_dtype)
        return self.forward(x, hidden)


class PositionEncoding(Part):
    """How positions enter the model. ``stage`` says where: 'embedding' (added to the token
    rows) or 'mixer' (applied to queries and keys inside the mixer)."""

    stage = "embedding"


class Block(Part):
    # True if ``forward`` takes and may return rows whose last sums are pending
    # (ops.kernels.PendingRows); a block that says False always gets plain float32 rows.
    takes_pending = False

    def forward(self, hidden, ctx: LayerContext):
        """hidden: [rows, width] float32 residual stream -> the same after this layer."""
        raise NotImplementedError

    def mixer_part(self) -> Mixer:
        raise NotImplementedError


# -- registries -----------------------------------------------------------------------------------
NORMS: dict[str, type] = {}
MIXERS: dict[str, type] = {}
FEED_FORWARDS: dict[str, type] = {}
POSITION_ENCODINGS: dict[str, type] = {}
BLOCKS: dict[str, type] = {}
_KINDS = {"norm": NORMS, "mixer": MIXERS, "feed_forward": FEED_FORWARDS, "position_encoding": POSITION_ENCODINGS, "block": BLOCKS}


def register_part(kind: str, name: str, cls: type) -> None:
    """kind: norm | mixer | feed_forward | position_encoding | block."""
    _KINDS[kind][name] = cls


def make_part(kind: str, name: str, **parameters):
    table = _KINDS[kind]
    if name not in table:
        raise KeyError(f"no {kind} named {name!r}; registered: {', '.join(sorted(table))}")
    return table[name](**parameters)

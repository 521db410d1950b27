"""The step function: one batch of (request, its next tokens) through the model and the cache.

The reference has three entry points (whole-prompt prefill of one sequence, decode of one token,
batched decode: engine/include/gpt2_gpu.h:64-68,89-90,161-165). Here there is one: portions of
prompts beside single decoded tokens, cut anywhere, run as one batch from the cache, with logits
returned only at the wanted places. Like the reference's calls it checks everything before it
changes anything (engine/src/gpt2_gpu_batch.cu:67-88), and a request's stored length grows only
after the step has been launched (engine/src/gpt2_gpu.cu:364)."""

from __future__ import annotations

from ..cache import CacheManager, OutOfPages
from .batch import BatchStaging, StepBatch, StepEntry, build_step_batch


class StepError(ValueError):
    """The batch cannot be run; nothing has been changed."""


class ModelRunner:
    def __init__(self, model, cache: CacheManager, device):
        self.model, self.cache, self.device = model, cache, device
        self.staging = BatchStaging(device) if device is not None else None
        self.steps_run = 0
        self.last_batch: StepBatch | None = None

    def validate(self, entries) -> None:
        if not entries:
            raise StepError("a step needs at least one entry")
        seen = set()
        vocab, limit = self.model.vocab_size, self.model.max_positions()
        for entry in entries:
            if entry.request_id in seen:
                raise StepError(f"request {entry.request_id!r} appears twice in one step")
            seen.add(entry.request_id)
            if not self.cache.has(entry.request_id):
                raise StepError(f"request {entry.request_id!r} is not open")
            n = len(entry.tokens)
            if n < 1:
                raise StepError(f"request {entry.request_id!r} brings no tokens")
            for token in entry.tokens:
                if not isinstance(token, (int,)) and not hasattr(token, "__index__"):
                    raise StepError(f"request {entry.request_id!r}: token {token!r} is not an integer")
                if not 0 <= int(token) < vocab:
                    raise StepError(f"request {entry.request_id!r}: token {token} is outside the vocabulary [0, {vocab})")
            length = self.cache.length(entry.request_id)
            if limit is not None and length + n > limit:
                raise StepError(f"request {entry.request_id!r}: {length} + {n} tokens exceed the model's {limit} positions")
            for w in entry.want:
                if not 0 <= int(w) < n:
                    raise StepError(f"request {entry.request_id!r}: wanted place {w} is not among its {n} tokens")

    def step(self, entries: list[StepEntry]):
        """Runs the entries as one batch. Returns float32 logits [wanted places, vocab] on the
        device (None if nothing is wanted), in the order of the entries and of each ``want``.
        Raises StepError / OutOfPages before anything has changed."""
        self.validate(entries)
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
            batch = build_step_batch(entries, self.cache, self.staging, vocab_size=self.model.vocab_size)
            logits = self.model.forward(batch, self.cache)
        except Exception:
            for request_id in reserved:
                self.cache.rollback(request_id)
            raise
        for entry in entries:
            self.cache.commit(entry.request_id, len(entry.tokens))
        self.steps_run += 1
        self.last_batch = batch
        return logits

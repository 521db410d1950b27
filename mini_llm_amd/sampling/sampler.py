"""Sampling on the device: packs the per-row parameters into one upload and calls the kernel."""

from __future__ import annotations

import numpy as np

from ..ops import kernels
from .params import SamplingParams


class Sampler:
    def __init__(self, staging):
        self._staging = staging  # engine.batch.BatchStaging: pinned upload buffers

    def sample(self, logits, params: list[SamplingParams], steps: list[int], token_slots=None, slot_of_row=None):
        """One token per row of ``logits`` (int32 on the device). steps[i] is the number of
        tokens row i's request has generated before this one. With ``token_slots`` (the cache's
        last-token slots) and ``slot_of_row`` (device int32) each token is also left in its
        request's slot."""
        n = logits.shape[0]
        if len(params) != n or len(steps) != n:
            raise ValueError("one SamplingParams and one step per row of logits")
        if all(p.greedy for p in params):
            return kernels.sample(logits, token_slots=token_slots, slot_of_row=slot_of_row)
        # [seeds as int64 | temperatures | top_ps | steps] in one int32 buffer, one copy
        flat = np.zeros(5 * n + (n & 1), dtype=np.int32)
        flat[: 2 * n].view(np.int64)[:] = [p.seed & 0x7FFFFFFFFFFFFFFF for p in params]
        flat[2 * n : 3 * n].view(np.float32)[:] = [max(p.temperature, 0.0) for p in params]
        flat[3 * n : 4 * n].view(np.float32)[:] = [p.top_p for p in params]
        flat[4 * n : 5 * n] = steps
        device = self._staging.upload(flat)
        import torch

        seeds = device[: 2 * n].view(torch.int64)
        temperatures = device[2 * n : 3 * n].view(torch.float32)
        top_ps = device[3 * n : 4 * n].view(torch.float32)
        return kernels.sample(logits, temperatures, top_ps, seeds, device[4 * n : 5 * n], token_slots=token_slots, slot_of_row=slot_of_row)

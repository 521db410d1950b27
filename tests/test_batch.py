"""The step's batch layout, without a GPU: the fast builder for decode steps gives exactly what
the general builder gives."""

import numpy as np

from mini_llm_amd.cache import CacheManager
from mini_llm_amd.engine.batch import DecodeBatchBuilder, StepEntry, build_step_batch
from mini_llm_amd.models.base import CacheGroupSpec


def test_decode_builder_matches_the_general_one():
    groups = [CacheGroupSpec("full", (0,), 2, 16, None), CacheGroupSpec("win", (1,), 1, 32, 24)]
    cache = CacheManager(groups, {}, num_pages={"full": 40, "win": 40}, page_size=16, max_requests=8, max_length=200)
    rng = np.random.default_rng(0)
    lengths = {}
    for name in "abcde":
        cache.open(name)
        lengths[name] = int(rng.integers(1, 120))
        cache.reserve(name, lengths[name]); cache.commit(name, lengths[name])
    builder = DecodeBatchBuilder(cache, 8)
    for live in (["a", "b", "c", "d", "e"], ["e", "b"], ["c"], ["a", "b", "c", "d", "e"]):  # shrinking, then growing again
        entries = [StepEntry(name, [int(rng.integers(0, 100))], [0], from_slot=(k % 2 == 0)) for k, name in enumerate(live)]
        for e in entries:
            cache.reserve(e.request_id, 1)
        general = build_step_batch(entries, cache, None, vocab_size=100, capacity=8)
        flat = builder.fill(entries)
        fast = builder.batch(flat, entries)
        for field in ("tokens", "positions", "token_request", "q_starts", "context_lens", "state_slots", "logit_rows", "token_sources", "logit_slots"):
            np.testing.assert_array_equal(getattr(fast, field), getattr(general, field), err_msg=field)
        for g in range(2):
            np.testing.assert_array_equal(fast.groups[g].block_tables, general.groups[g].block_tables)
            np.testing.assert_array_equal(fast.groups[g].slots, general.groups[g].slots)
        assert (fast.token_sources[: len(live)] >= 0).tolist() == [k % 2 == 0 for k in range(len(live))]
        assert (fast.n_tokens, fast.n_requests, fast.n_logit_rows, fast.max_q_len) == (8, 8, 8, 1)
        for e in entries:
            cache.commit(e.request_id, 1)

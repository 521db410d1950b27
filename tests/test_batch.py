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


def test_short_portions_are_laid_out_first_and_logit_rows_keep_the_given_order():
    groups = [CacheGroupSpec("full", (0,), 2, 16, None)]
    cache = CacheManager(groups, {}, num_pages=40, page_size=16, max_requests=8, max_length=200)
    for name, length in (("a", 30), ("b", 0), ("c", 7), ("d", 50), ("e", 3)):
        cache.open(name)
        if length:
            cache.reserve(name, length); cache.commit(name, length)
    entries = [
        StepEntry("b", list(range(100, 120)), [19]),     # a long portion, given first
        StepEntry("a", [7], [0]),                        # a decoded token
        StepEntry("d", list(range(200, 209)), []),       # nine tokens: long, nothing wanted
        StepEntry("c", [1, 2, 3, 4, 5, 6, 7, 8], [7, 0]),  # eight tokens: still short
        StepEntry("e", [9], [0], from_slot=True),
    ]
    for e in entries:
        cache.reserve(e.request_id, len(e.tokens))
    batch = build_step_batch(entries, cache, None, vocab_size=1000)
    assert batch.request_ids == ["a", "c", "e", "b", "d"]
    assert (batch.short_requests, batch.short_rows, batch.max_q_len) == (3, 10, 20)
    assert batch.q_starts.tolist() == [0, 1, 9, 10, 30, 39]
    assert batch.tokens.tolist() == [7] + [1, 2, 3, 4, 5, 6, 7, 8] + [9] + list(range(100, 120)) + list(range(200, 209))
    assert batch.context_lens.tolist() == [30, 7, 3, 0, 50]
    assert batch.positions.tolist() == [30] + list(range(7, 15)) + [3] + list(range(20)) + list(range(50, 59))
    assert batch.token_request.tolist() == [0] + [1] * 8 + [2] + [3] * 20 + [4] * 9
    # logits come in the order of the entries as given and of each want
    assert batch.logit_rows.tolist() == [29, 0, 8, 1, 9]
    slot = {name: cache.requests[name].state_slot for name in "abcde"}
    assert batch.logit_slots.tolist() == [slot["b"], slot["a"], slot["c"], slot["c"], slot["e"]]
    assert batch.state_slots.tolist() == [slot[n] for n in "acebd"]
    # the rows of the batch, listed in the order of the entries as given
    given = batch.rows_in_order_of([e.request_id for e in entries])
    assert given == list(range(10, 30)) + [0] + list(range(30, 39)) + list(range(1, 9)) + [9]
    assert np.asarray(batch.tokens)[given].tolist() == [t for e in entries for t in e.tokens]
    assert batch.token_sources.tolist() == [-1] * 9 + [slot["e"]] + [-1] * 29
    for i, name in enumerate("acebd"):
        pages = cache.block_table(name, 0)
        assert batch.groups[0].block_tables[i, : len(pages)].tolist() == list(pages)


def test_a_padded_shape_of_portions():
    # the same five entries as above, laid out in the padded shape (16 rows of short portions, 64 of long ones, 2 long
    # requests) that batches of many shapes share: padding rows belong to nobody, the long portions begin at row 16
    groups = [CacheGroupSpec("full", (0,), 2, 16, None)]
    cache = CacheManager(groups, {}, num_pages=40, page_size=16, max_requests=8, max_length=200)
    for name, length in (("a", 30), ("b", 0), ("c", 7), ("d", 50), ("e", 3)):
        cache.open(name)
        if length:
            cache.reserve(name, length); cache.commit(name, length)
    entries = [
        StepEntry("b", list(range(100, 120)), [19]),
        StepEntry("a", [7], [0]),
        StepEntry("d", list(range(200, 209)), []),
        StepEntry("c", [1, 2, 3, 4, 5, 6, 7, 8], [7, 0]),
        StepEntry("e", [9], [0], from_slot=True),
    ]
    for e in entries:
        cache.reserve(e.request_id, len(e.tokens))
    batch = build_step_batch(entries, cache, None, vocab_size=1000, pad=(16, 64, 2))
    assert (batch.n_tokens, batch.n_requests, batch.n_logit_rows) == (80, 18, 18)
    assert (batch.short_requests, batch.short_rows, batch.max_q_len, batch.max_total_len) == (16, 16, 64, 200)
    assert batch.tokens.tolist() == [7] + [1, 2, 3, 4, 5, 6, 7, 8] + [9] + [-1] * 6 + list(range(100, 120)) + list(range(200, 209)) + [-1] * 35
    assert batch.token_request.tolist() == [0] + [1] * 8 + [2] + [-1] * 6 + [16] * 20 + [17] * 9 + [-1] * 35
    assert batch.q_starts.tolist() == [0, 1, 9] + [10] * 13 + [16, 36, 45]
    assert batch.context_lens.tolist() == [30, 7, 3] + [-1] * 13 + [0, 50]   # -1: a padding request
    slot = {name: cache.requests[name].state_slot for name in "abcde"}
    assert batch.state_slots.tolist() == [slot["a"], slot["c"], slot["e"]] + [-1] * 13 + [slot["b"], slot["d"]]
    assert batch.positions.tolist()[:10] == [30] + list(range(7, 15)) + [3] and batch.positions.tolist()[16:45] == list(range(20)) + list(range(50, 59))
    assert batch.logit_rows.tolist() == [35, 0, 8, 1, 9] + [0] * 13
    assert batch.logit_slots.tolist() == [slot["b"], slot["a"], slot["c"], slot["c"], slot["e"]] + [-1] * 13
    assert batch.token_sources.tolist() == [-1] * 9 + [slot["e"]] + [-1] * 70
    table, slots = batch.groups[0].block_tables, batch.groups[0].slots
    for at, name in ((0, "a"), (1, "c"), (2, "e"), (16, "b"), (17, "d")):
        pages = cache.block_table(name, 0)
        assert table[at, : len(pages)].tolist() == list(pages)
    assert (table[3:16] == -1).all() and (np.asarray(slots)[10:16] == -1).all() and (np.asarray(slots)[45:] == -1).all()
    assert (np.asarray(slots)[:10] >= 0).all() and (np.asarray(slots)[16:45] >= 0).all()
    # a batch that does not fit the shape is refused
    import pytest

    with pytest.raises(ValueError):
        build_step_batch(entries, cache, None, vocab_size=1000, pad=(16, 64, 1))
    with pytest.raises(ValueError):
        build_step_batch(entries, cache, None, vocab_size=1000, pad=(0, 64, 2))


def test_hot_shapes_beyond_the_kept_graphs_are_not_captured_at_every_turn():
    # more shapes of batch than graphs are kept, taking turns: a shape that loses its graph starts counting again, so
    # the number of captures stays far below the number of steps (a capture costs some forty steps' time)
    from mini_llm_amd.engine import step as step_module
    from mini_llm_amd.engine.step import ModelRunner

    class NoModel:
        vocab_size = 100

        def short_portion(self):
            return 8

        def all_graph_safe(self):
            return True

        def decode_reaches(self):
            return []

    groups = [CacheGroupSpec("full", (0,), 2, 16, None)]
    cache = CacheManager(groups, {}, num_pages=8, page_size=16, max_requests=4, max_length=64)
    runner = ModelRunner(NoModel(), cache, None, portion_graph_after=2)
    # one shape more than graphs are kept: portions of 10, 74, 138, ... tokens fall in padded shapes 64 rows apart
    shapes = [[StepEntry("r", [0] * n, [n - 1])] for n in range(10, 10 + 64 * (step_module.PORTION_GRAPHS_KEPT + 1), 64)]
    rounds = 40
    for _ in range(rounds):
        for entries in shapes:
            runner._portion_graph_for(entries)
    steps = rounds * len(shapes)
    assert runner.portion_graphs_made <= steps // 4, (runner.portion_graphs_made, steps)
    assert len(runner._portion_graphs) <= step_module.PORTION_GRAPHS_KEPT
    # as many shapes as graphs are kept: each is captured once and kept
    runner = ModelRunner(NoModel(), cache, None, portion_graph_after=2)
    for _ in range(rounds):
        for entries in shapes[:-1]:
            runner._portion_graph_for(entries)
    assert runner.portion_graphs_made == step_module.PORTION_GRAPHS_KEPT and runner.portion_graphs_dropped == 0

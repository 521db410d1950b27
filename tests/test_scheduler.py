"""The scheduler's decisions, without a GPU, against a fake step function that records the
composition of every step (the reference tests its scheduler the same way:
pytorch/tests/test_scheduler.py with pytorch/tests/batch_fakes.py). A sequence's tokens are
prompt[0] + 1, + 2, ... so that every sequence is recognisable."""

import time

import pytest

from mini_llm_amd.cache import CacheManager
from mini_llm_amd.engine.background import SchedulerThread
from mini_llm_amd.engine.scheduler import Request, Scheduler
from mini_llm_amd.models.base import CacheGroupSpec
from mini_llm_amd.sampling import SamplingParams


class FakeExecutor:
    def __init__(self, num_pages=16, page_size=4, max_requests=8, positions=64, vocab=10_000):
        self.cache = CacheManager([CacheGroupSpec("full", (0,), 1, 16, None)], {}, num_pages=num_pages,
                                  page_size=page_size, max_requests=max_requests, max_length=positions)
        self.page_size, self._positions, self._vocab = page_size, positions, vocab
        self.steps = []          # per step: [(request_id, tokens fed, wants)]
        self.fed = {}
        self.closed = []
        self.fail_next_run = False
        self.total_pages = num_pages

    def max_positions(self):
        return self._positions

    def check_prompt(self, tokens):
        if len(tokens) > self._positions:
            raise ValueError("prompt too long")
        if any(not 0 <= t < self._vocab for t in tokens):
            raise ValueError("token outside the vocabulary")

    def can_open(self):
        return self.cache.can_open()

    def open(self, request_id):
        self.cache.open(request_id)
        self.fed[request_id] = []

    def close(self, request_id):
        self.cache.close(request_id)
        self.closed.append(request_id)

    def length(self, request_id):
        return self.cache.length(request_id)

    def pages_needed(self, request_id, n_new):
        return self.cache.pages_needed(request_id, n_new)

    def free_pages(self):
        return self.cache.free_pages()

    def run(self, entries, sampling, steps):
        if self.fail_next_run:
            self.fail_next_run = False
            raise RuntimeError("boom")
        out, k = [], 0
        self.steps.append([(e.request_id, list(e.tokens), list(e.want)) for e in entries])
        for e in entries:
            self.cache.reserve(e.request_id, len(e.tokens))
        for e in entries:
            self.cache.commit(e.request_id, len(e.tokens))
            self.fed[e.request_id] += e.tokens
            if e.want:
                assert e.want == [len(e.tokens) - 1]
                base, generated = self.fed[e.request_id][0], steps[k]
                if generated:  # what was fed back must be what was sampled
                    assert self.fed[e.request_id][-generated:] == [base + i for i in range(1, generated + 1)], "wrong token fed back"
                out.append(base + generated + 1)
                k += 1
        self.cache.check_invariants()
        return out

    def all_free(self):
        return self.cache.free_pages() == [self.total_pages] and not self.cache.requests


class Sink:
    def __init__(self):
        self.tokens, self.finish, self.error = [], None, None

    def emit(self, token, finish):
        self.tokens.append(token)
        if finish is not None:
            assert self.finish is None, "finished twice"
            self.finish = finish

    def fail(self, message):
        self.error = message


def submit(scheduler, prompt, max_new=4, eos=None, **kw):
    sink = Sink()
    request = Request(list(prompt), on_token=sink.emit, on_error=sink.fail, max_new_tokens=max_new, eos_token_id=eos, **kw)
    scheduler.submit(request)
    return sink, request


def composition(executor):
    return [[(r, len(t)) for r, t, _ in step] for step in executor.steps]


def test_one_request_generates_until_length():
    ex = FakeExecutor()
    s = Scheduler(ex)
    sink, _ = submit(s, [100, 5, 6], max_new=4)
    s.run_until_idle()
    assert sink.tokens == [101, 102, 103, 104] and sink.finish == "length" and sink.error is None
    assert composition(ex) == [[(0, 3)], [(0, 1)], [(0, 1)], [(0, 1)]]
    assert ex.steps[0][0][2] == [2] and ex.all_free()
    assert not s.step()  # nothing to do


def test_finish_reasons_and_their_order():
    ex = FakeExecutor(positions=8)
    s = Scheduler(ex)
    stop, _ = submit(s, [100, 1], max_new=10, eos=103)
    context, _ = submit(s, [200, 1, 2, 3, 4], max_new=10)          # 5 + 3 >= 8
    first, _ = submit(s, [300], max_new=1)                          # the first token already ends it
    both, _ = submit(s, [400, 1, 2, 3, 4, 5, 6], max_new=1, eos=401)  # stop, context and length at once
    cl, _ = submit(s, [500, 1, 2, 3, 4, 5, 6], max_new=1)           # context and length at once
    s.run_until_idle()
    assert (stop.tokens, stop.finish) == ([101, 102, 103], "stop")  # the finishing token is emitted
    assert (context.tokens, context.finish) == ([201, 202, 203], "context")
    assert (first.tokens, first.finish) == ([301], "length")
    assert both.finish == "stop" and cl.finish == "context"
    assert ex.all_free()


def test_max_batch_and_admission_when_one_ends():
    ex = FakeExecutor()
    s = Scheduler(ex, max_batch=2)
    sinks = [submit(s, [100 * (i + 1)], max_new=2 + i)[0] for i in range(3)]
    s.run_until_idle()
    assert composition(ex) == [[(0, 1), (1, 1)], [(0, 1), (1, 1)], [(1, 1), (2, 1)], [(2, 1)], [(2, 1)], [(2, 1)]]
    assert [x.tokens for x in sinks] == [[101, 102], [201, 202, 203], [301, 302, 303, 304]]
    assert all(len(step) <= 2 for step in ex.steps)


def test_prompts_are_cut_into_portions_under_the_token_budget():
    ex = FakeExecutor(num_pages=32)
    s = Scheduler(ex, max_tokens_per_step=8)
    a, _ = submit(s, [100] + [1] * 19, max_new=3)                   # 20 tokens: 8 + 8 + 4
    s.step(); s.step()
    b, _ = submit(s, [200] + [2] * 9, max_new=2)                    # arrives while a is in its prompt
    s.run_until_idle()
    assert composition(ex) == [
        [(0, 8)], [(0, 8)],
        [(0, 4), (1, 4)],          # a's last portion, the rest of the budget to b
        [(0, 1), (1, 6)],          # a decodes beside b's portion: one mixed batch
        [(0, 1), (1, 1)],
    ]
    assert ex.steps[1][0][2] == [] and ex.steps[2][0][2] == [3] and ex.steps[2][1][2] == []
    assert a.tokens == [101, 102, 103] and b.tokens == [201, 202]
    assert all(sum(n for _, n in step) <= 8 for step in composition(ex))


def test_decodes_come_before_prompt_portions_in_the_budget():
    ex = FakeExecutor(num_pages=32)
    s = Scheduler(ex, max_tokens_per_step=4)
    a, _ = submit(s, [100], max_new=6)
    s.step()
    b, _ = submit(s, [200] + [0] * 8, max_new=1)
    s.run_until_idle()
    assert composition(ex)[1:4] == [[(0, 1), (1, 3)], [(0, 1), (1, 3)], [(0, 1), (1, 3)]]


def test_max_prefills_per_step():
    ex = FakeExecutor()
    s = Scheduler(ex, max_prefills_per_step=1)
    for i in range(3):
        submit(s, [100 * (i + 1)], max_new=3)
    s.run_until_idle()
    assert composition(ex)[:3] == [[(0, 1)], [(0, 1), (1, 1)], [(0, 1), (1, 1), (2, 1)]]


def test_the_head_of_the_queue_is_not_overtaken():
    ex = FakeExecutor(num_pages=4, page_size=4)
    s = Scheduler(ex)
    a, _ = submit(s, [100] + [0] * 8, max_new=6)                    # 3 pages, grows into the 4th
    s.step()
    big, _ = submit(s, [200] + [0] * 10, max_new=1)                 # its first page does not fit beside a
    small, _ = submit(s, [300], max_new=1)                          # would fit, but must wait its turn
    s.step(); s.step()
    assert all(r == 0 for step in ex.steps for r, _, _ in step)
    assert s.stats()["waiting"] == 2 and small.tokens == []
    s.run_until_idle()
    assert big.tokens == [201] and small.tokens == [301] and a.finish == "length"
    first_big = next(i for i, step in enumerate(ex.steps) if any(r == 1 for r, _, _ in step))
    first_small = next(i for i, step in enumerate(ex.steps) if any(r == 2 for r, _, _ in step))
    assert first_big <= first_small and ex.all_free()


def test_when_pages_run_out_the_youngest_is_preempted_and_recomputed():
    outputs = {}
    for pages in (64, 6):                                           # plenty / so few that decoding runs out
        ex = FakeExecutor(num_pages=pages, page_size=4)
        s = Scheduler(ex)
        sinks = [submit(s, [100 * (i + 1)] + [0] * 6, max_new=12)[0] for i in range(3)]
        s.run_until_idle()
        outputs[pages] = [x.tokens for x in sinks]
        assert all(x.finish == "length" and x.error is None for x in sinks)
        assert ex.all_free()
        if pages == 6:
            assert s.stats()["preemptions"] > 0
            # the oldest request is never the victim: it appears in every step until it ends
            last = max(i for i, step in enumerate(ex.steps) if any(r == 0 for r, _, _ in step))
            assert all(any(r == 0 for r, _, _ in step) for step in ex.steps[: last + 1])
            # a recompute feeds the prompt and what was generated, as one prompt again
            assert any(len(t) > 7 for step in ex.steps for _, t, _ in step)
        else:
            assert s.stats()["preemptions"] == 0
    assert outputs[6] == outputs[64] == [[100 * (i + 1) + k for k in range(1, 13)] for i in range(3)]


def test_a_request_that_cannot_fit_the_pool_fails_alone():
    ex = FakeExecutor(num_pages=3, page_size=4)
    s = Scheduler(ex)
    big, _ = submit(s, [100] + [0] * 10, max_new=8)                 # 11 + 8 tokens > 12
    ok, _ = submit(s, [200, 0], max_new=3)
    s.run_until_idle()
    assert big.error is not None and "pages" in big.error and big.finish is None
    assert ok.tokens == [201, 202, 203] and ok.error is None and ex.all_free()


def test_cancel_waiting_and_running():
    ex = FakeExecutor()
    s = Scheduler(ex, max_batch=1)
    a, ra = submit(s, [100], max_new=10)
    b, rb = submit(s, [200], max_new=10)
    s.step(); s.step()
    rb.cancel()                                                     # still waiting: never prefilled
    ra.cancel()                                                     # running: leaves before the next step
    assert s.step() is False
    assert a.tokens == [101, 102] and b.tokens == [] and ex.all_free()
    assert all(r == 0 for step in ex.steps for r, _, _ in step)


def test_engine_error_fails_all_running_and_the_scheduler_goes_on():
    ex = FakeExecutor()
    s = Scheduler(ex)
    a, _ = submit(s, [100], max_new=5)
    b, _ = submit(s, [200], max_new=5)
    s.step()
    ex.fail_next_run = True
    assert s.step() is True
    assert a.error == "boom" and b.error == "boom" and ex.all_free()
    c, _ = submit(s, [300], max_new=2)
    s.run_until_idle()
    assert c.tokens == [301, 302] and c.error is None


def test_a_bad_prompt_fails_only_its_request():
    ex = FakeExecutor(vocab=1000, positions=16)
    s = Scheduler(ex)
    bad_token, _ = submit(s, [100, 5000])
    empty, _ = submit(s, [])
    too_long, _ = submit(s, [1] * 17)
    good, _ = submit(s, [300], max_new=2)
    s.run_until_idle()
    assert "vocabulary" in bad_token.error and "no tokens" in empty.error and "long" in too_long.error
    assert good.tokens == [301, 302] and ex.all_free()


def test_a_raising_callback_drops_only_its_request():
    ex = FakeExecutor()
    s = Scheduler(ex)
    good, _ = submit(s, [100], max_new=3)
    def boom(token, finish):
        raise RuntimeError("consumer gone")
    s.submit(Request([200], on_token=boom, on_error=lambda m: None, max_new_tokens=3))
    s.run_until_idle()
    assert good.tokens == [101, 102, 103] and ex.all_free()
    assert sum(1 for step in ex.steps for r, _, _ in step if r == 1) == 1


def test_sampling_parameters_and_step_numbers_reach_the_engine():
    seen = []
    class Recording(FakeExecutor):
        def run(self, entries, sampling, steps):
            seen.append((list(sampling), list(steps)))
            return super().run(entries, sampling, steps)
    ex = Recording()
    s = Scheduler(ex)
    params = SamplingParams(temperature=0.8, top_p=0.9, seed=4)
    submit(s, [100, 1, 2], max_new=3, sampling=params)
    s.run_until_idle()
    assert seen == [([params], [0]), ([params], [1]), ([params], [2])]


def test_stats():
    ex = FakeExecutor()
    s = Scheduler(ex)
    submit(s, [100, 1, 2], max_new=3)
    submit(s, [200], max_new=2)
    s.run_until_idle()
    stats = s.stats()
    assert stats["tokens"] == 5 and stats["prefills"] == 2 and stats["running"] == 0 and stats["waiting"] == 0
    assert stats["steps"] == 3 and stats["decode_steps"] == 2 and stats["mean_batch_size"] == 1.5
    assert stats["tokens_per_step"] == pytest.approx((4 + 2 + 1) / 3) and stats["preemptions"] == 0


def test_thread_idles_processes_and_stops():
    ex = FakeExecutor()
    s = SchedulerThread(Scheduler(ex, max_batch=1))
    s.start()
    assert s.is_running()
    with pytest.raises(RuntimeError):
        s.start()
    sink, _ = submit(s, [100], max_new=3)
    deadline = time.time() + 5
    while sink.finish is None and time.time() < deadline:
        time.sleep(0.01)
    assert sink.tokens == [101, 102, 103]
    s.stop()
    assert not s.is_running() and ex.all_free()
    late, _ = submit(s, [200])                     # after the end: refused at once
    assert late.error is not None and "shutting down" in late.error


def test_shutdown_fails_what_is_live_and_what_waits():
    ex = FakeExecutor()
    s = Scheduler(ex, max_batch=1)
    live, _ = submit(s, [100], max_new=5)
    waiting, _ = submit(s, [200], max_new=5)
    s.step()
    s.shutdown("closing")
    assert live.tokens == [101] and live.error == "closing" and waiting.error == "closing" and waiting.tokens == []
    assert ex.all_free() and not s.has_work() and s.step() is False


def test_options_are_checked():
    with pytest.raises(ValueError):
        Scheduler(FakeExecutor(), max_batch=0)
    with pytest.raises(ValueError):
        Scheduler(FakeExecutor(), max_tokens_per_step=0)


# --- one step ahead -----------------------------------------------------------------------------
class AheadExecutor(FakeExecutor):
    """The fake with launch / collect: a launched step is worked off at once, as a device would in
    launch order, and leaves each sampled token in its request's slot; the host sees the tokens
    at collect. It records how many steps were launched while another had not been collected."""

    def __init__(self, *args, **kw):
        super().__init__(*args, **kw)
        self.slot = {}
        self.uncollected = 0
        self.launched_ahead = 0
        self.fail_next_collect = False

    def launch(self, entries, sampling, steps):
        for e in entries:
            if e.from_slot:
                assert e.tokens == [0] and e.want == [0]
                e.tokens = [self.slot[e.request_id]]
        tokens = self.run(entries, sampling, steps)
        sampled = [e.request_id for e in entries if e.want]
        self.slot.update(zip(sampled, tokens))
        assert self.uncollected <= 1, "more than one step ahead"
        self.launched_ahead += self.uncollected
        self.uncollected += 1
        return tokens

    def collect(self, handle):
        self.uncollected -= 1
        if self.fail_next_collect:
            self.fail_next_collect = False
            raise RuntimeError("late boom")
        return handle


def test_a_step_is_launched_before_the_one_before_it_is_read():
    ex = AheadExecutor()
    s = Scheduler(ex)
    a, _ = submit(s, [100, 5, 6], max_new=5)
    b, _ = submit(s, [200], max_new=3)
    s.run_until_idle()
    assert a.tokens == [101, 102, 103, 104, 105] and b.tokens == [201, 202, 203]
    assert (a.finish, b.finish) == ("length", "length") and ex.all_free()
    # an end by length is counted ahead: no step runs for a token that nobody wants
    assert composition(ex) == [[(0, 3), (1, 1)], [(0, 1), (1, 1)], [(0, 1), (1, 1)], [(0, 1)], [(0, 1)]]
    assert ex.launched_ahead == 4 and s.stats()["dropped_tokens"] == 0
    assert s.stats()["tokens"] == 8 and s.stats()["prefills"] == 2 and s.stats()["decode_steps"] == 4


def test_an_end_token_is_seen_one_step_late_and_the_token_past_it_is_dropped():
    ex = AheadExecutor()
    s = Scheduler(ex)
    stop, _ = submit(s, [100, 1], max_new=10, eos=103)
    other, _ = submit(s, [200], max_new=6)
    s.run_until_idle()
    assert (stop.tokens, stop.finish) == ([101, 102, 103], "stop")
    assert other.tokens == [201, 202, 203, 204, 205, 206] and ex.all_free()
    assert sum(1 for step in ex.steps for r, _, _ in step if r == 0) == 4   # one step more than its 3 tokens
    assert s.stats()["dropped_tokens"] == 1 and s.stats()["tokens"] == 9


def test_ends_by_context_are_counted_ahead():
    ex = AheadExecutor(positions=8)
    s = Scheduler(ex)
    context, _ = submit(s, [200, 1, 2, 3, 4], max_new=10)            # 5 + 3 >= 8
    s.run_until_idle()
    assert (context.tokens, context.finish) == ([201, 202, 203], "context")
    assert composition(ex) == [[(0, 5)], [(0, 1)], [(0, 1)]] and s.stats()["dropped_tokens"] == 0


@pytest.mark.parametrize("seed", range(6))
def test_one_step_ahead_delivers_what_step_by_step_delivers(seed):
    """Random requests (prompt lengths, limits, end tokens, arrival times) in a pool so small that
    requests are preempted: the same tokens and finish reasons either way, and every page back."""
    import random

    def play(executor, **kw):
        rng = random.Random(seed)
        s = Scheduler(executor, max_batch=4, max_tokens_per_step=rng.choice([4, 7, 64]), **kw)
        sinks = []
        for i in range(12):
            prompt = [500 * (i + 1)] + [rng.randrange(50) for _ in range(rng.randrange(0, 14))]
            max_new = rng.randrange(1, 16)
            eos = prompt[0] + rng.randrange(1, 20) if rng.random() < 0.5 else None
            sinks.append(submit(s, prompt, max_new=max_new, eos=eos)[0])
            for _ in range(rng.randrange(0, 4)):
                s.step()
        s.run_until_idle()
        return s, sinks

    plain_s, plain = play(FakeExecutor(num_pages=9, page_size=4, positions=24))
    ex = AheadExecutor(num_pages=9, page_size=4, positions=24)
    ahead_s, ahead = play(ex)
    assert [(x.tokens, x.finish, x.error) for x in ahead] == [(x.tokens, x.finish, x.error) for x in plain]
    assert all(x.finish is not None for x in plain)
    assert ex.all_free() and ex.launched_ahead > 0
    assert ahead_s.stats()["tokens"] == plain_s.stats()["tokens"]
    if seed == 0:
        assert plain_s.stats()["preemptions"] > 0 and ahead_s.stats()["preemptions"] > 0


def test_a_plan_that_must_preempt_reads_the_step_in_flight_first():
    ex = AheadExecutor(num_pages=6, page_size=4)
    s = Scheduler(ex)
    sinks = [submit(s, [100 * (i + 1)] + [0] * 6, max_new=12)[0] for i in range(3)]
    s.run_until_idle()
    assert [x.tokens for x in sinks] == [[100 * (i + 1) + k for k in range(1, 13)] for i in range(3)]
    assert s.stats()["preemptions"] > 0 and ex.all_free()


def test_cancel_with_a_step_in_flight():
    ex = AheadExecutor()
    s = Scheduler(ex)
    a, ra = submit(s, [100], max_new=10)
    b, _ = submit(s, [200], max_new=4)
    s.step(); s.step()                                               # the second step is in flight
    assert a.tokens == [101]
    ra.cancel()
    s.run_until_idle()
    assert a.tokens == [101] and b.tokens == [201, 202, 203, 204] and ex.all_free()
    assert s.stats()["dropped_tokens"] == 1


def test_an_error_at_collect_fails_the_running_requests():
    ex = AheadExecutor()
    s = Scheduler(ex)
    a, _ = submit(s, [100], max_new=5)
    s.step(); s.step()
    ex.fail_next_collect = True
    assert s.step() is True
    assert a.error == "late boom" and ex.all_free()
    ex.uncollected = 0                                               # the failed step's successor is forgotten
    c, _ = submit(s, [300], max_new=2)
    s.run_until_idle()
    assert c.tokens == [301, 302] and c.error is None


def test_step_ahead_can_be_switched_off():
    ex = AheadExecutor()
    s = Scheduler(ex, step_ahead=False)
    a, _ = submit(s, [100], max_new=3)
    s.run_until_idle()
    assert a.tokens == [101, 102, 103] and ex.launched_ahead == 0 and ex.uncollected == 0


def test_thread_runs_one_step_ahead_and_stops_with_a_step_in_flight():
    ex = AheadExecutor()
    scheduler = Scheduler(ex, max_batch=2)
    s = SchedulerThread(scheduler)
    s.start()
    sinks = [submit(s, [100 * (i + 1)], max_new=5, eos=(203 if i == 1 else None))[0] for i in range(3)]
    deadline = time.time() + 5
    while any(x.finish is None for x in sinks) and time.time() < deadline:
        time.sleep(0.01)
    assert [x.tokens for x in sinks] == [[101, 102, 103, 104, 105], [201, 202, 203], [301, 302, 303, 304, 305]]
    assert [x.finish for x in sinks] == ["length", "stop", "length"]
    deadline = time.time() + 5
    while scheduler.has_work() and time.time() < deadline:   # the token past the end token is collected and dropped
        time.sleep(0.01)
    assert ex.all_free() and ex.launched_ahead > 0 and scheduler.stats()["dropped_tokens"] == 1
    slow_collect = ex.collect
    ex.collect = lambda handle: (time.sleep(0.01), slow_collect(handle))[1]
    endless, _ = submit(s, [400], max_new=None)                       # 63 tokens at 10 ms each
    while len(endless.tokens) < 3:
        time.sleep(0.001)
    s.stop()                                                          # whatever is in flight is forgotten
    assert endless.error is not None and "shutting down" in endless.error and ex.all_free()


def test_a_submit_that_races_shutdown_is_always_answered():
    # another thread submits while this one shuts down: every request either reached the queue before it was drained
    # or hears the message at once; none is left in a queue nobody looks at again
    import threading

    for trial in range(20):
        scheduler = Scheduler(FakeExecutor())
        sinks, started = [], threading.Event()

        def feed():
            for i in range(400):
                sinks.append(submit(scheduler, [100 + i, 1])[0])
                if i == 20:
                    started.set()

        thread = threading.Thread(target=feed)
        thread.start()
        started.wait()
        scheduler.shutdown("closing")
        thread.join()
        assert len(sinks) == 400 and all(sink.error == "closing" for sink in sinks), trial
        assert not scheduler.has_work()

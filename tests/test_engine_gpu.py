"""Generation through the entry point, the step function's checks, cache reuse, long decoding,
the first tokens of a sequence: the engine against the plain implementation."""

import math

import numpy as np
import pytest
import torch

import plain_gpt2
from conftest import random_tokens

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def engines(model_dirs):
    from mini_llm_amd.engine.engine import Engine, EngineOptions

    cache = {}

    def get(name, dtype="float32", **options):
        key = (name, dtype, tuple(sorted(options.items())))
        if key not in cache:
            cache[key] = Engine(model_dirs[name][0], EngineOptions(dtype=dtype, **options))
        return cache[key]

    return get


def plain_check_greedy(config, weights, prompt, generated, margin, stored=plain_gpt2._keep):
    """Every generated token must be (within margin) the plain implementation's argmax."""
    tokens = list(prompt)
    for token in generated:
        logits = plain_gpt2.forward(config, weights, tokens, stored=stored)[-1]
        assert logits[token] >= logits.max() - margin, f"token {token} at length {len(tokens)}: {logits[token]} < {logits.max()}"
        tokens.append(token)


def test_greedy_generation_matches_plain_f32(model_dirs, engines):
    # three requests with prompts of 5, 17 and 33 ids, 16 greedy tokens each
    _, config, weights = model_dirs["A"]
    prompts = [random_tokens(1 + i, n, config["vocab_size"]) for i, n in enumerate((5, 17, 33))]
    out = engines("A").generate(prompts, max_new_tokens=16)
    for prompt, generated in zip(prompts, out):
        assert generated == plain_gpt2.greedy(config, weights, prompt, 16)


@pytest.mark.parametrize("name", ["A", "B"])
def test_greedy_generation_bf16(model_dirs, engines, name):
    _, config, weights = model_dirs[name]
    rounded = plain_gpt2.bf16_weights(weights)
    prompts = [random_tokens(1 + i, n, config["vocab_size"]) for i, n in enumerate((5, 17, 33))]
    out = engines(name, "bfloat16").generate(prompts, max_new_tokens=16)
    for prompt, generated in zip(prompts, out):
        assert len(generated) == 16
        plain_check_greedy(config, rounded, prompt, generated, margin=0.03, stored=plain_gpt2.stored_as_bf16)


def host_uniform(seed, step, index):
    """The sampler's counter-based generator, on the host (mini_llm_amd/csrc/sampling.hip)."""
    m = (1 << 64) - 1
    z = (seed + 0x9E3779B97F4A7C15 * (step + 1) + 0xD1B54A32D192ED03 * (index + 1)) & m
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & m
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & m
    z = z ^ (z >> 31)
    return float((np.float32(z >> 41) + np.float32(0.5)) * np.float32(1.0 / 8388608.0))   # 23 bits, in 32-bit like the kernel


def test_temperature_sampling_in_chunks_beside_decodes(model_dirs, engines):
    # prompts of 1, 9 and 40 ids prefilled in 8-token portions beside ongoing decodes, 20 new
    # tokens each at temperature 0.8; every draw is checked against the generator on the host
    _, config, weights = model_dirs["B"]
    vocab = config["vocab_size"]
    prompts = [random_tokens(3 + i, n, vocab) for i, n in enumerate((1, 9, 40))]
    engine = engines("B", "float32", max_tokens_per_step=8)
    out = engine.generate(prompts, max_new_tokens=20, temperature=0.8, seed=4)
    assert engine.stats()["tokens_per_step"] <= 8
    assert out != engines("B").generate(prompts, max_new_tokens=20)  # it really samples
    for i, (prompt, generated) in enumerate(zip(prompts, out)):
        assert len(generated) == 20
        tokens = list(prompt)
        for step, token in enumerate(generated):
            logits = plain_gpt2.forward(config, weights, tokens)[-1]
            noise = np.array([-math.log(-math.log(host_uniform(4 + i, step, v))) for v in range(vocab)])
            score = (logits - logits.max()) / 0.8 + noise
            assert score[token] >= score.max() - 1e-3, f"request {i} step {step}: token {token} is not the draw"
            tokens.append(token)
    # the same seeds give the same tokens in another batch composition
    alone = engines("B").generate([prompts[2]], max_new_tokens=20, temperature=0.8, seed=6)
    assert alone[0] == out[2]


def test_sampled_rows_are_drawn_inside_the_captured_decode_step(model_dirs):
    # Three requests decode side by side through the scheduler, one greedily, one at temperature 0.7, one at 1.3 with a
    # nucleus: the captured step draws the tokens itself (the rows' parameters and counts of tokens drawn lie in its
    # device buffer, and the counts move on with the batch), so that between two steps of the same requests nothing is
    # copied. Every token is checked against the plain implementation and the generator on the host.
    from mini_llm_amd.engine.engine import Engine, EngineOptions
    from mini_llm_amd.engine.scheduler import Request
    from mini_llm_amd.sampling import SamplingParams

    folder, config, weights = model_dirs["A"]
    vocab = config["vocab_size"]
    engine = Engine(folder, EngineOptions(dtype="float32", max_sessions=4))
    prompts = [random_tokens(20 + i, n, vocab) for i, n in enumerate((6, 11, 3))]
    hows = [SamplingParams(), SamplingParams(temperature=0.7, seed=5), SamplingParams(temperature=1.3, top_p=0.6, seed=9)]
    new_tokens = 40
    out = [[] for _ in prompts]
    for i, (prompt, how) in enumerate(zip(prompts, hows)):
        engine.submit(Request(prompt, on_token=lambda token, finish, i=i: out[i].append(token), on_error=lambda message: pytest.fail(message),
                              max_new_tokens=new_tokens, sampling=how))
    engine.scheduler.run_until_idle()
    drawn = [g for key, g in engine.runner._graphs.items() if len(key) == 4]
    assert len(drawn) == 1 and drawn[0].draws
    # three requests of 9 to 51 tokens cross a page edge (64 tokens a page) never, and finish together: the batch is
    # brought from the host once, and once more at most for what the scheduler's first decode step finds
    assert drawn[0].uploads <= 2, drawn[0].uploads
    assert engine.runner.graph_steps >= new_tokens - 2
    for i, (prompt, how, generated) in enumerate(zip(prompts, hows, out)):
        assert len(generated) == new_tokens
        tokens = list(prompt)
        for step, token in enumerate(generated):
            logits = plain_gpt2.forward(config, weights, tokens)[-1]
            if how.greedy:
                assert token == int(np.argmax(logits)), (i, step)
            else:
                noise = np.array([-math.log(-math.log(host_uniform(how.seed, step, v))) for v in range(vocab)])
                score = (logits - logits.max()) / how.temperature + noise
                if how.top_p < 1.0:   # outside the nucleus nothing is drawn (a little slack for rounding at its edge)
                    p = plain_gpt2.softmax(logits / how.temperature)
                    assert p[p > p[token] * (1 + 1e-4)].sum() < how.top_p + 1e-4, (i, step)
                    surely_inside = np.array([p[p > p[v] * (1 - 1e-4)].sum() - p[v] < how.top_p - 1e-3 for v in range(vocab)])
                    score = np.where(surely_inside | (np.arange(vocab) == token), score, -np.inf)   # it beats all that are surely inside
                assert score[token] >= score.max() - 1e-3, f"request {i} step {step}: token {token} is not the draw"
            tokens.append(token)
    engine.close()


def test_top_p_generation_stays_in_the_nucleus(model_dirs, engines):
    _, config, weights = model_dirs["A"]
    prompt = random_tokens(9, 12, config["vocab_size"])
    (generated,) = engines("A").generate([prompt], max_new_tokens=12, temperature=1.5, top_p=0.3, seed=11)
    tokens = list(prompt)
    for token in generated:
        p = plain_gpt2.softmax(plain_gpt2.forward(config, weights, tokens)[-1] / 1.5)
        # kept if the mass of strictly more likely tokens is below top_p (a little slack for rounding)
        assert p[p > p[token] * (1 + 1e-4)].sum() < 0.3 + 1e-4
        tokens.append(token)


def test_eos_and_context_limits(model_dirs, engines):
    _, config, weights = model_dirs["B"]
    prompt = random_tokens(5, 10, config["vocab_size"])
    free = plain_gpt2.greedy(config, weights, prompt, 6)
    (out,) = engines("B").generate([prompt], max_new_tokens=6, eos_token_id=free[3])
    assert out == free[: free.index(free[3]) + 1]
    # 60 + 4 = n_positions: generation stops at the context's end; a longer prompt is cut from the left
    long_prompt = random_tokens(6, 60, config["vocab_size"])
    (out,) = engines("B").generate([long_prompt], max_new_tokens=50)
    assert len(out) == 50 and len(long_prompt[-14:]) + 50 == 64
    (out,) = engines("B").generate([long_prompt[:60]], max_new_tokens=4)
    assert out == plain_gpt2.greedy(config, weights, long_prompt[:60], 4)


def test_sessions_and_forward_last(model_dirs, engines):
    _, config, weights = model_dirs["A"]
    engine = engines("A")
    tokens = random_tokens(7, 30, config["vocab_size"])
    import replay

    ref = plain_gpt2.forward(config, weights, tokens)
    tol = replay.F32_TOL
    np.testing.assert_allclose(engine.forward_last(tokens), ref[-1], **tol)
    with engine.open_session() as session:
        np.testing.assert_allclose(session.prefill(tokens[:1]), ref[0], **tol)   # the very first token
        np.testing.assert_allclose(session.decode(tokens[1]), ref[1], **tol)
        np.testing.assert_allclose(session.prefill(tokens[2:20]), ref[19], **tol)
        for i in range(20, 30):
            np.testing.assert_allclose(session.decode(tokens[i]), ref[i], **tol)
        assert session.length() == 30
    with pytest.raises(RuntimeError, match="closed"):
        session.decode(1)


def test_the_reference_schedulers_four_calls(model_dirs, engines):
    # try_take_cache / prefill_greedy / decode_batch / release_cache (pytorch/src/mini_llm/batch_api.py)
    _, config, weights = model_dirs["A"]
    engine = engines("A", "float32", max_sessions=3)
    prompts = [random_tokens(20 + i, n, config["vocab_size"]) for i, n in enumerate((3, 11, 26))]
    handles = [engine.try_take_cache() for _ in prompts]
    assert engine.try_take_cache() is None  # all taken: None, no waiting
    last = [engine.prefill_greedy(h, p) for h, p in zip(handles, prompts)]
    got = [[t] for t in last]
    for _ in range(7):
        last = engine.decode_batch(handles, last)
        for g, t in zip(got, last):
            g.append(t)
    for h in handles:
        engine.release_cache(h)
    assert got == [plain_gpt2.greedy(config, weights, p, 8) for p in prompts]
    handle = engine.try_take_cache()
    assert handle is not None
    engine.release_cache(handle)


def test_step_checks_everything_before_it_changes_anything(model_dirs, engines):
    from mini_llm_amd.cache import OutOfPages
    from mini_llm_amd.engine import StepEntry, StepError

    engine = engines("B", "float32", max_sessions=4, max_tokens=64)  # one page
    a, b = engine.try_take_cache(), engine.try_take_cache()
    engine.runner.step([StepEntry(a, [1, 2, 3], [2])])
    free = engine.cache.free_pages()
    bad = [
        [StepEntry(a, [4], [0]), StepEntry(b, [1000], [0])],      # a token outside the vocabulary
        [StepEntry(a, [4], [0]), StepEntry(a, [5], [0])],         # a request twice
        [StepEntry(a, [4], [0]), StepEntry("nobody", [5], [0])],  # an unknown request
        [StepEntry(a, [4] * 62, [0])],                            # 3 + 62 > n_positions
        [StepEntry(a, [], [])],                                   # no tokens
        [StepEntry(a, [4, 5], [2])],                              # a wanted place that is not there
        [],
    ]
    for entries in bad:
        with pytest.raises(StepError):
            engine.runner.step(entries)
        assert engine.cache.length(a) == 3 and engine.cache.length(b) == 0 and engine.cache.free_pages() == free
    # a holds the only page: a's next token fits on it, b's does not, and neither is taken
    with pytest.raises(OutOfPages):
        engine.runner.step([StepEntry(a, [4], [0]), StepEntry(b, [5] * 5, [0])])
    assert engine.cache.length(a) == 3 and engine.cache.free_pages() == free
    engine.cache.check_invariants()
    engine.release_cache(a); engine.release_cache(b)


def test_used_pages_give_the_same_bits_as_fresh_ones(model_dirs, engines):
    # the reference's reset test: a cache used by a longer sequence gives bit-equal results
    # (engine/tests/test_gpt2_gpu.c:266-289)
    _, config, _ = model_dirs["A"]
    from mini_llm_amd.engine.engine import Engine, EngineOptions

    tokens = random_tokens(30, 70, config["vocab_size"])
    fresh = Engine(model_dirs["A"][0], EngineOptions(dtype="float32", max_sessions=2, max_tokens=128))
    first = fresh.forward_last(tokens)
    other = fresh.forward_last(random_tokens(31, 128, config["vocab_size"]))  # fills every page with something else
    again = fresh.forward_last(tokens)
    assert (first == again).all() and not (first == other).all()


def test_long_decoding_and_page_edges(model_dirs, tmp_path):
    # 40 tokens at once, then 540 one by one across nine page edges, against the whole sequence
    import replay

    folder, config, weights = model_dirs["C"]
    requests = {"long": random_tokens(40, 580, config["vocab_size"])}
    collector = replay.prefill_then_decode(requests, tail=540)
    for dtype in ("float32", "bfloat16"):
        got = collector.gather(replay.run_trace(folder, dtype, collector.steps, tmp_path / dtype, 640))
        replay.compare(got, replay.plain_logits(config, weights, requests, bf16=(dtype == "bfloat16")), **replay.tolerance(dtype))


@pytest.mark.parametrize("page_size", [16, 32, 128])
def test_other_page_sizes(model_dirs, tmp_path, page_size):
    import replay

    folder, config, weights = model_dirs["A"]
    requests = {f"r{i}": random_tokens(50 + i, n, config["vocab_size"]) for i, n in enumerate((33, 128, 17, 65))}
    collector = replay.mixed(requests, seed=page_size)
    max_tokens = replay.peak_tokens(collector, page=max(64, page_size))
    got = collector.gather(replay.run_trace(folder, "float32", collector.steps, tmp_path / "o", max_tokens, page_size=page_size))
    replay.compare(got, replay.plain_logits(config, weights, requests), **replay.F32_TOL)


def test_trace_run_refuses_bad_folders(tmp_path, model_dirs):
    import json
    import subprocess
    import sys

    import replay

    folder, config, weights = model_dirs["A"]
    broken = tmp_path / "broken"
    broken.mkdir()
    (broken / "config.json").write_text(json.dumps(config))
    w = dict(weights)
    del w["h.0.ln_1.bias"]
    plain_gpt2.write_safetensors(broken / "model.safetensors", w)
    cmd = [sys.executable, str(replay.ROOT / "bin" / "trace_run"), "--model", str(broken), "--dtype", "float32", "--out", str(tmp_path / "o"), "--max-tokens", "64"]
    done = subprocess.run(cmd, input="", capture_output=True, text=True, timeout=300)
    assert done.returncode != 0 and "missing (1): h.0.ln_1.bias" in done.stderr


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_graph_replays_match_eager_steps(model_dirs, dtype):
    # decode steps replayed from a captured graph, with eager steps (prompt portions, other batch
    # sizes) and synchronisations between the replays; every replay is checked against the same
    # step run without graphs and against the plain implementation
    from mini_llm_amd.engine import StepEntry
    from mini_llm_amd.engine.engine import Engine, EngineOptions

    folder, config, weights = model_dirs["C"]
    vocab = config["vocab_size"]
    seqs = {name: random_tokens(60 + i, n, vocab) for i, (name, n) in enumerate((("a", 150), ("b", 90), ("c", 131), ("d", 70)))}
    import replay

    ref = replay.plain_logits(config, weights, seqs, bf16=(dtype == "bfloat16"))
    tol = replay.tolerance(dtype)
    results = {}
    for use_graphs in (True, False):
        engine = Engine(folder, EngineOptions(dtype=dtype, max_sessions=8, max_tokens=1024, use_graphs=use_graphs))
        handles = {name: engine.try_take_cache() for name in seqs}
        fed = {name: 0 for name in seqs}
        got = {name: {} for name in seqs}

        def run(step):
            entries = [StepEntry(handles[name], seqs[name][fed[name] : fed[name] + n], [n - 1]) for name, n in step]
            logits = engine.runner.step(entries).cpu().numpy()
            for row, (name, n) in zip(logits, step):
                fed[name] += n
                got[name][fed[name] - 1] = row

        run([("a", 100), ("b", 40)])
        for i in range(30):
            run([("a", 1), ("b", 1)])                     # bucket of 2, replayed
            if i == 5:
                run([("c", 77)])                          # an eager step in between
            if i > 5:
                run([("c", 1)])                           # bucket of 1
            if i % 7 == 0:
                torch.cuda.synchronize()
            if i == 12:
                run([("d", 50), ("a", 1)])                # mixed: eager
            if i > 12 and i % 2:
                run([("a", 1), ("b", 1), ("c", 1)])       # bucket of 4 with a padding row
        assert (engine.runner.graph_steps > 0) == use_graphs
        results[use_graphs] = got
        for name in seqs:
            for position, row in got[name].items():
                np.testing.assert_allclose(row, ref[name][position], err_msg=f"{name} {position} graphs={use_graphs}", **tol)
    for name in seqs:
        assert results[True][name].keys() == results[False][name].keys()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_captured_portion_steps_match_eager_steps(model_dirs, dtype):
    # steps with portions of prompts whose padded shape of batch keeps coming (the rows of short portions in steps of 16, of
    # long portions in steps of 64, long requests in powers of two) are
    # captured (here at the second time, by option) and replayed from then on: here the same shapes come with other requests, at other
    # depths of the cache and with other places wanted, with decode replays, eager steps of other shapes and
    # synchronisations between them; every step is checked against the plain implementation, with and without graphs
    from mini_llm_amd.engine import StepEntry
    from mini_llm_amd.engine.engine import Engine, EngineOptions

    folder, config, weights = model_dirs["C"]
    vocab = config["vocab_size"]
    seqs = {name: random_tokens(80 + i, 190, vocab) for i, name in enumerate("abcdef")}
    import replay

    ref = replay.plain_logits(config, weights, seqs, bf16=(dtype == "bfloat16"))
    tol = replay.tolerance(dtype)
    for use_graphs in (True, False):
        engine = Engine(folder, EngineOptions(dtype=dtype, max_sessions=8, max_tokens=2048, use_graphs=use_graphs, portion_graph_after=2))
        handles = {name: engine.try_take_cache() for name in seqs}
        fed = {name: 0 for name in seqs}
        checked = 0

        def run(step):
            nonlocal checked
            entries = [StepEntry(handles[name], seqs[name][fed[name] : fed[name] + n], list(want)) for name, n, want in step]
            logits = engine.runner.step(entries).cpu().numpy()
            row = 0
            for name, n, want in step:
                for w in want:
                    np.testing.assert_allclose(logits[row], ref[name][fed[name] + w], err_msg=f"{name} {fed[name] + w} graphs={use_graphs}", **tol)
                    row += 1
                    checked += 1
                fed[name] += n

        # shape X: 30 + 1 tokens, two requests, two places wanted; shape Y: 40 + 20 + 2 tokens, three wanted
        run([("a", 30, [29]), ("b", 1, [0])])                     # X, first time: eager
        run([("c", 40, [39]), ("d", 20, [5]), ("e", 2, [1])])     # Y, first time: eager
        run([("b", 30, [0]), ("a", 1, [0])])                      # X again, the long portion first: captured here
        run([("e", 40, [7]), ("c", 20, [19]), ("f", 2, [0])])     # Y again: captured here
        run([("a", 1, [0]), ("b", 1, [0])])                       # a decode step between
        torch.cuda.synchronize()
        run([("f", 30, [10]), ("d", 1, [0])])                     # X replayed, deeper in the cache
        run([("d", 33, [32])])                                    # another shape: eager
        run([("a", 40, [39]), ("b", 20, [0]), ("d", 2, [1])])     # Y replayed
        run([("c", 30, [29]), ("e", 1, [0])])                     # X replayed
        torch.cuda.synchronize()
        run([("f", 40, [0]), ("e", 20, [19]), ("c", 2, [0])])     # Y replayed
        run([("a", 30, [3]), ("f", 1, [0])])                      # X replayed
        assert checked == 2 * 5 + 3 * 4 + 2 + 1
        assert engine.runner.portion_graph_steps == (7 if use_graphs else 0)
        # shape Z: a portion of 131 tokens (the products and the prompt attention for many rows) beside a single decoded
        # token and a portion of two; replayed at two depths of the cache, the second one starting inside a page and
        # inside a tile of 32 keys
        for name in "abc":
            engine.release_cache(handles[name])
            handles[name] = engine.try_take_cache()
            fed[name] = 0
        run([("a", 40, []), ("b", 50, [49]), ("c", 3, [])])       # some history first
        run([("a", 131, [130]), ("b", 1, [0]), ("c", 2, [1])])    # Z: eager
        for name in "ab":
            engine.release_cache(handles[name])
            handles[name] = engine.try_take_cache()
            fed[name] = 0
        run([("b", 131, [130]), ("c", 1, [0]), ("a", 2, [0])])    # Z again: captured here, the long portion from an empty cache
        run([("a", 43, [42]), ("c", 5, [])])                      # depths 45 (a), 11 (c); 43 + 5 tokens fall in X's padded shape: replayed
        run([("a", 131, [7]), ("b", 1, [0]), ("c", 2, [1])])      # Z replayed: the long portion starts at 45, inside a page and a tile
        assert engine.runner.portion_graph_steps == (10 if use_graphs else 0)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_step_takes_the_kernels_it_is_meant_to(tmp_path, dtype):
    # Logits stay right whichever kernels compute them; which ones a step took shows only in the library's launch
    # counts (the reference pins its launches per step the same way: engine/tests/test_gpt2_gpu_batch.c:170-194,
    # engine/tests/test_gpt2_gpu_half.c:108-118). Two layers at GPT-2 small's width, steps run eagerly.
    import json

    from mini_llm_amd.config import config_from_dict
    from mini_llm_amd.engine import StepEntry
    from mini_llm_amd.engine.engine import Engine, EngineOptions
    from mini_llm_amd.ops import kernels

    raw = {"architectures": ["GPT2LMHeadModel"], "n_layer": 2, "n_embd": 768, "n_head": 12, "n_inner": 3072, "vocab_size": 9001,
           "n_positions": 512, "layer_norm_epsilon": 1e-5, "activation_function": "gelu_new"}
    engine = Engine.from_random(config_from_dict(raw), 3, EngineOptions(dtype=dtype, max_sessions=8, use_graphs=False))
    layers = raw["n_layer"]
    handles = [engine.try_take_cache() for _ in range(8)]
    rng = np.random.default_rng(0)
    before = kernels.launch_counts()
    engine.runner.step([StepEntry(handles[0], rng.integers(0, 9001, 300).tolist(), [299])])
    prompt_step = kernels.launches_since(before)
    for h in handles[1:]:
        engine.runner.step([StepEntry(h, rng.integers(0, 9001, 20).tolist(), [])])
    before = kernels.launch_counts()
    logits = engine.runner.step([StepEntry(h, [int(rng.integers(0, 9001))], [0]) for h in handles])
    decode_step = kernels.launches_since(before)
    before = kernels.launch_counts()
    kernels.sample(logits)
    assert kernels.launches_since(before) == {"sample": 1}
    if dtype == "bfloat16":
        # a portion of 300 rows: the four products of a layer stream their operands into LDS, the attention is the streaming one
        assert prompt_step.get("gemm_stream") == 4 * layers, prompt_step
        assert prompt_step.get("attention_prefill_stream") == layers and "attention_prefill" not in prompt_step, prompt_step
        # eight single tokens: the two layer kernels a layer, and embedding, final norm and head around them
        assert decode_step == {"embed": 1, "decode_attention_half": layers, "decode_mlp_half": layers, "pending_layernorm": 1,
                               "gemm_tiled": 1}, decode_step
        assert sum(decode_step.values()) == 2 * layers + 3
    else:
        assert prompt_step.get("gemm_tiled") == 4 * layers + 1 and "gemm_stream" not in prompt_step, prompt_step
        assert prompt_step.get("attention_prefill_stream") == layers and "attention_prefill" not in prompt_step, prompt_step
        # the separate kernels: norm, q/k/v with the cache write, attention, output product cut along K, norm taking its
        # partial products, up product, down product cut along K; the final norm takes the last partial products
        assert decode_step == {"embed": 1, "layernorm": 1, "pending_layernorm": 2 * layers, "gemm_skinny": 4 * layers,
                               "attention_decode": layers, "gemm_tiled": 1}, decode_step
        assert sum(decode_step.values()) == 7 * layers + 3
    engine.close()


@pytest.mark.parametrize("use_graphs", [True, False])
def test_decoding_changes_kernels_where_the_sequences_grow_long(model_dirs, monkeypatch, use_graphs):
    # Past a length that the mixer names, a decode step runs its attention through the separate kernels instead of the
    # layer kernel (whose block walks all keys of a row alone); a captured step is kept for either range. The length is
    # brought down to 48 here so that two requests cross it one after the other, and every step is checked against the
    # plain implementation; the tokens a choosing step leaves are the argmax of those logits.
    import replay
    from mini_llm_amd.engine import StepEntry
    from mini_llm_amd.engine.engine import Engine, EngineOptions
    from mini_llm_amd.ops import kernels
    from mini_llm_amd.parts.attention import CausalSelfAttention

    monkeypatch.setattr(kernels, "DECODE_LAYER_REACHES", (48, 48))
    # and the separate attention kernel cuts each row's keys into runs of 16, a block each, as it does for thousands of
    # keys: the counters the blocks go by serve launch after launch, replayed from a graph or not
    monkeypatch.setattr(kernels, "DECODE_MIN_PART_FEW", 16)
    monkeypatch.setattr(CausalSelfAttention, "decode_reaches", (48,))
    folder, config, weights = model_dirs["A"]
    seqs = {"a": random_tokens(7, 70, config["vocab_size"]), "b": random_tokens(8, 62, config["vocab_size"])}
    ref = replay.plain_logits(config, weights, seqs, bf16=True)
    tol = replay.tolerance("bfloat16")
    engine = Engine(folder, EngineOptions(dtype="bfloat16", max_sessions=4, use_graphs=use_graphs))
    handles = {name: engine.try_take_cache() for name in seqs}
    engine.runner.step([StepEntry(handles["a"], seqs["a"][:40], []), StepEntry(handles["b"], seqs["b"][:32], [])])
    fed = {"a": 40, "b": 32}
    kinds = []
    for i in range(30):
        before = kernels.launch_counts()
        entries = [StepEntry(handles[name], [seqs[name][fed[name]]], [0]) for name in seqs]
        logits = engine.runner.step(entries).cpu().numpy()
        kinds.append("decode_attention_half" in kernels.launches_since(before))
        for row, name in zip(logits, seqs):
            np.testing.assert_allclose(row, ref[name][fed[name]], err_msg=f"{name} {fed[name]}", **tol)
            fed[name] += 1
    assert kernels._arrival_counters and all((counters == 0).all() for counters in kernels._arrival_counters.values())
    if use_graphs:
        assert sorted(key[2] for key in engine.runner._graphs) == [48, config["n_positions"]]
    else:  # a's newest token is the 41st..70th: the first eight steps stay within 48
        assert kinds == [True] * 8 + [False] * 22
    # the same through steps that choose their tokens: from a's 45th token on, across the change
    for name in seqs:
        engine.release_cache(handles[name])
        handles[name] = engine.try_take_cache()
    first = engine.runner.step([StepEntry(handles["a"], seqs["a"][:44], [43]), StepEntry(handles["b"], seqs["b"][:36], [35])], choose=True)
    chosen = [first.tolist()]
    for _ in range(9):
        chosen.append(engine.runner.step([StepEntry(handles[name], [0], [0], from_slot=True) for name in seqs], choose=True).tolist())
    rounded = plain_gpt2.bf16_weights(weights)
    for j, (name, start) in enumerate((("a", 44), ("b", 36))):
        tokens = list(seqs[name][:start])
        for step in chosen:
            plain_check_greedy(config, rounded, tokens, [step[j]], margin=0.03, stored=plain_gpt2.stored_as_bf16)
            tokens.append(step[j])
    engine.close()


def test_no_garbage_collection_while_a_step_is_captured():
    # the collector may finalise another engine's captured graphs, and giving memory back inside a capture aborts the
    # process: it is off from the start of a capture to its end, and as it was again afterwards
    import gc

    from mini_llm_amd.engine.step import _capture

    class Runner:
        device = "cuda:0"
        seen = []

        def forward(self, batch):
            self.seen.append(gc.isenabled())
            return torch.ones(4, device="cuda:0") * 2

    runner = Runner()
    assert gc.isenabled()
    graph, logits = _capture(runner, None)
    assert runner.seen == [True, False] and gc.isenabled()   # the eager run first, then the capture
    graph.replay()
    torch.cuda.synchronize()
    assert logits.tolist() == [2.0, 2.0, 2.0, 2.0]
    gc.disable()
    try:
        _capture(runner, None)
        assert not gc.isenabled()   # left as it was found
    finally:
        gc.enable()


def test_queued_decoding_gives_the_same_tokens(model_dirs, engines):
    # step n+1 is launched before the host has read token n; the tokens must be those of the
    # step-by-step calls and of the plain implementation (the reference's queued mode:
    # engine/tests/test_gpt2_gpu_greedy.c:59-322)
    _, config, weights = model_dirs["A"]
    engine = engines("A", "float32", max_sessions=5)
    prompts = [random_tokens(70 + i, n, config["vocab_size"]) for i, n in enumerate((4, 19, 60))]
    handles = [engine.try_take_cache() for _ in prompts]
    got = [[engine.prefill_greedy(h, p)] for h, p in zip(handles, prompts)]
    engine.decode_batch_enqueue(handles)
    engine.decode_batch_enqueue(handles)          # two steps in flight
    for _ in range(10):
        engine.decode_batch_enqueue(handles)
        for g, t in zip(got, engine.take()):
            g.append(t)
    for _ in range(2):
        for g, t in zip(got, engine.take()):
            g.append(t)
    with pytest.raises(RuntimeError, match="no step is queued"):
        engine.take()
    # a sequence leaves, the others go on; then a step-by-step call continues from the same state
    engine.release_cache(handles[0])
    engine.decode_batch_enqueue(handles[1:])
    for g, t in zip(got[1:], engine.take()):
        g.append(t)
    last = engine.decode_batch(handles[1:], [g[-1] for g in got[1:]])
    for g, t in zip(got[1:], last):
        g.append(t)
    for h in handles[1:]:
        engine.release_cache(h)
    assert got[0] == plain_gpt2.greedy(config, weights, prompts[0], 13)
    assert got[1] == plain_gpt2.greedy(config, weights, prompts[1], 15)
    assert got[2] == plain_gpt2.greedy(config, weights, prompts[2], 15)
    for _ in range(engine.MAX_QUEUED):
        h = engine.try_take_cache()
        engine.prefill_greedy(h, prompts[0])
        engine.decode_batch_enqueue([h])
        engine.release_cache(h)
    h = engine.try_take_cache()
    engine.prefill_greedy(h, prompts[0])
    with pytest.raises(RuntimeError, match="queued already"):
        engine.decode_batch_enqueue([h])
    engine.release_cache(h)
    while engine._queued:
        engine.take()
    # a request that was never sampled has no token in its slot (the slot still holds its previous
    # owner's): queueing a step for it is refused, and nothing has changed
    from mini_llm_amd.engine import StepError

    fresh = engine.try_take_cache()
    with pytest.raises(StepError, match="no token has been sampled"):
        engine.decode_batch_enqueue([fresh])
    with engine.open_session() as session:
        session.prefill(prompts[0])                                  # logits to the host, nothing sampled
        with pytest.raises(StepError, match="no token has been sampled"):
            engine.decode_batch_enqueue([session._handle])
        assert session.length() == len(prompts[0])
    assert engine.prefill_greedy(fresh, prompts[0]) == got[0][0]
    engine.decode_batch_enqueue([fresh])
    assert engine.take() == [got[0][1]]
    engine.release_cache(fresh)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_queued_decoding_of_many_sequences_side_by_side_without_copies(model_dirs, dtype):
    # 40 sequences decode for 70 steps, queued: the captured step chooses its tokens itself and moves its batch on by
    # one token on the device, so between two steps nothing is copied to the device unless a sequence has reached a new
    # page (all prompts have the same length here: every 16th step); by option the step's requests go through the layers
    # in two groups side by side (branches of the captured graph). The tokens must be the plain implementation's.
    from mini_llm_amd.engine.engine import Engine, EngineOptions

    folder, config, weights = model_dirs["A"]
    engine = Engine(folder, EngineOptions(dtype=dtype, max_sessions=40, page_size=16, decode_lanes_from=32))
    prompts = [random_tokens(900 + i, 21, config["vocab_size"]) for i in range(40)]
    handles = [engine.try_take_cache() for _ in prompts]
    got = [[engine.prefill_greedy(h, p)] for h, p in zip(handles, prompts)]
    steps = 70
    engine.decode_batch_enqueue(handles)
    for _ in range(steps - 1):
        engine.decode_batch_enqueue(handles)
        for g, t in zip(got, engine.take()):
            g.append(t)
    for g, t in zip(got, engine.take()):
        g.append(t)
    graph, = [g for key, g in engine.runner._graphs.items() if key[:2] == (64, True)]
    assert graph.lanes is not None and len(graph.lanes.cuts(64)) == 2
    assert engine.runner.graph_steps == steps and graph.uploads <= 2 + steps // 16, graph.uploads
    rounded = plain_gpt2.bf16_weights(weights) if dtype == "bfloat16" else None
    for i in range(0, 40, 3):
        if dtype == "float32":
            assert got[i] == plain_gpt2.greedy(config, weights, prompts[i], steps + 1), i
        else:
            plain_check_greedy(config, rounded, prompts[i], got[i], margin=0.03, stored=plain_gpt2.stored_as_bf16)
    # a sequence leaves and the rest go on: the device's batch no longer stands for them, so it is brought anew
    engine.release_cache(handles[0])
    before = graph.uploads
    engine.decode_batch_enqueue(handles[1:])
    tokens = engine.take()
    assert graph.uploads == before + 1 and len(tokens) == 39
    if dtype == "float32":
        assert tokens[2] == plain_gpt2.greedy(config, weights, prompts[3], steps + 2)[-1]
    engine.close()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_one_step_ahead_gives_the_tokens_of_step_by_step(model_dirs, engines, dtype):
    # nine requests in a pool that holds about three of them (requests wait, and some are preempted
    # and recomputed), prompts in portions of 24 tokens beside decodes, an end token for every
    # other request, greedy and sampled: the scheduler that launches a step before it has read the
    # one before must deliver exactly what the step-by-step one delivers, and drop what it
    # computed past an end token
    from mini_llm_amd.engine.scheduler import Request
    from mini_llm_amd.sampling import SamplingParams

    _, config, weights = model_dirs["A"]
    vocab = config["vocab_size"]
    prompts = [random_tokens(200 + i, n, vocab) for i, n in enumerate((3, 40, 11, 64, 7, 29, 50, 2, 33))]
    results = {}
    for ahead in (False, True):
        engine = engines("A", dtype, max_sessions=4, max_tokens=256, max_tokens_per_step=24, step_ahead=ahead)
        for temperature in (0.0, 0.9):
            if temperature == 0.0 and not ahead:
                free = engine.generate(prompts, max_new_tokens=24)
                assert engine.stats()["preemptions"] >= 1  # the pool is that small
                ends = [tokens[5 + i] if i % 2 == 0 else None for i, tokens in enumerate(free)]
            outputs, errors = [[] for _ in prompts], []
            for i, prompt in enumerate(prompts):
                def emit(token, finish, i=i):
                    outputs[i].append((token, finish))
                engine.submit(Request(prompt, on_token=emit, on_error=errors.append, max_new_tokens=24, eos_token_id=ends[i],
                                      sampling=SamplingParams(temperature=temperature, seed=31 + i)))
            before = engine.stats()
            engine.scheduler.run_until_idle()
            after = engine.stats()
            results[ahead, temperature] = outputs
            assert not errors
            assert all(o and o[-1][1] is not None and all(f is None for _, f in o[:-1]) for o in outputs)
            assert engine.cache.free_pages() == [engine.cache.pools[0].num_pages] and not engine.cache.requests
            if ahead and temperature == 0.0:
                assert after["dropped_tokens"] - before["dropped_tokens"] >= 1
                assert any(f == "stop" for o in outputs for _, f in o)
            if not ahead:
                assert after["dropped_tokens"] == 0
    for temperature in (0.0, 0.9):
        assert results[True, temperature] == results[False, temperature]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_captured_mixed_steps_take_tokens_from_slots(model_dirs, dtype):
    # The default serving path: the scheduler one step ahead (decode rows take their token from the last-token slot)
    # with steps of prompt portions beside decodes replayed from captured graphs once their shape of batch has come
    # twice. Long prompts under a small budget keep one shape coming (three decodes beside a portion that fills the
    # budget); the pool is so small that requests are preempted and recomputed. Every request's tokens must be the
    # plain implementation's greedy ones.
    from mini_llm_amd.engine.engine import Engine, EngineOptions
    from mini_llm_amd.engine.step import _PortionGraph

    folder, config, weights = model_dirs["C"]
    vocab = config["vocab_size"]
    prompts = [random_tokens(300 + i, n, vocab) for i, n in enumerate((150, 151, 149, 152, 150, 148, 153, 150))]
    engine = Engine(folder, EngineOptions(dtype=dtype, max_sessions=4, max_tokens=42 * 16, page_size=16, max_tokens_per_step=32,
                                          portion_graph_after=2, step_ahead=True))
    runner = engine.runner
    replayed_with_slot_rows, mixed_replays = 0, 0
    plain_step = runner.step

    def watched_step(entries, *args, **kwargs):
        nonlocal replayed_with_slot_rows, mixed_replays
        before = runner.portion_graph_steps
        logits = plain_step(entries, *args, **kwargs)
        if runner.portion_graph_steps > before:
            mixed_replays += 1
            if any(e.from_slot for e in entries) and any(len(e.tokens) > 1 for e in entries):
                replayed_with_slot_rows += 1
        return logits

    runner.step = watched_step
    generated = engine.generate(prompts, max_new_tokens=20)
    stats = engine.stats()
    assert stats["preemptions"] >= 1, stats                 # the pool is that small
    assert runner.portion_graph_steps > 0 and runner.portion_graphs_made >= 1
    assert replayed_with_slot_rows >= 3, (replayed_with_slot_rows, mixed_replays, runner.portion_graphs_made)
    assert engine.cache.free_pages() == [engine.cache.pools[0].num_pages] and not engine.cache.requests
    if dtype == "float32":
        for prompt, new in zip(prompts, generated):
            assert new == plain_gpt2.greedy(config, weights, prompt, 20)
    else:
        rounded = plain_gpt2.bf16_weights(weights)
        for prompt, new in zip(prompts, generated):
            assert len(new) == 20
            plain_check_greedy(config, rounded, prompt, new, margin=0.03, stored=plain_gpt2.stored_as_bf16)
    engine.close()


def test_cache_sized_by_memory(model_dirs):
    from mini_llm_amd.engine.engine import Engine, EngineOptions

    folder, config, weights = model_dirs["A"]
    per_token = config["n_layer"] * 2 * config["n_embd"] * 4
    engine = Engine(folder, EngineOptions(dtype="float32", cache_gib=300 * 64 * per_token / (1 << 30), page_size=64, max_sessions=4))
    assert engine.cache.free_pages() == [300]
    prompt = random_tokens(9, 12, config["vocab_size"])
    assert engine.generate([prompt], max_new_tokens=6)[0] == plain_gpt2.greedy(config, weights, prompt, 6)
    with pytest.raises(ValueError):
        Engine(folder, EngineOptions(dtype="float32", cache_gib=1.0, max_tokens=1024))


def test_the_callers_longest_sequence_narrows_the_models_own(model_dirs):
    from mini_llm_amd.engine import StepEntry, StepError
    from mini_llm_amd.engine.engine import Engine, EngineOptions
    from mini_llm_amd.engine.scheduler import Request

    folder, config, weights = model_dirs["A"]     # 128 positions
    engine = Engine(folder, EngineOptions(dtype="float32", max_sessions=2, max_length=40, page_size=16))
    assert engine.cache.max_length == 40 and engine.cache.max_blocks() == 3 and engine.cache.free_pages() == [2 * 3]
    wider = Engine(folder, EngineOptions(dtype="float32", max_sessions=2, max_length=4096))
    assert wider.cache.max_length == 128           # never beyond the model's positions
    wider.close()
    prompt = random_tokens(90, 30, config["vocab_size"])
    handle = engine.try_take_cache()
    with pytest.raises(StepError, match="exceed the 40 positions"):
        engine.runner.step([StepEntry(handle, prompt + prompt, [0])])
    assert engine.cache.length(handle) == 0
    engine.release_cache(handle)
    got = []
    engine.submit(Request(prompt, on_token=lambda token, finish: got.append((token, finish)), on_error=got.append, max_new_tokens=30))
    engine.scheduler.run_until_idle()
    assert [token for token, _ in got] == plain_gpt2.greedy(config, weights, prompt, 10) and got[-1][1] == "context"
    engine.close()


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_random_workloads_through_the_scheduler_match_plain_greedy(model_dirs, engines, seed):
    # random prompt lengths and lengths to generate, portions under a small budget, a pool that holds
    # a few requests (so some wait and some are preempted and recomputed): whatever the scheduler
    # does, every request gets the plain implementation's greedy tokens
    name = "ABC"[seed]   # (C: heads of 48, whose short portions go through the kernel that walks request by request)
    _, config, weights = model_dirs[name]
    rng = np.random.default_rng(50 + seed)
    limit = config["n_positions"]
    prompts, new = [], []
    for i in range(14):
        n = int(rng.integers(1, limit // 2))
        prompts.append(random_tokens(700 + 20 * seed + i, n, config["vocab_size"]))
        new.append(int(rng.integers(1, min(24, limit - n) + 1)))
    engine = engines(name, "float32", max_sessions=5, max_tokens=(2 if seed < 2 else 1) * limit, page_size=16, max_tokens_per_step=int(rng.integers(8, 40)))
    before = engine.stats()["preemptions"]
    outputs = [engine.generate([prompt], max_new_tokens=n)[0] for prompt, n in zip(prompts[:2], new[:2])]   # alone
    from mini_llm_amd.engine.scheduler import Request

    together, errors = [[] for _ in prompts], []
    for i, (prompt, n) in enumerate(zip(prompts, new)):
        engine.submit(Request(prompt, on_token=lambda token, finish, i=i: together[i].append(token), on_error=errors.append,
                              max_new_tokens=n))
    engine.scheduler.run_until_idle()
    assert not errors
    if seed < 2:
        assert engine.stats()["preemptions"] > before   # the pool is that small (the third model's requests grow too little for it)
    for i, (prompt, n) in enumerate(zip(prompts, new)):
        assert together[i] == plain_gpt2.greedy(config, weights, prompt, n), f"request {i} ({len(prompt)} prompt tokens, {n} new)"
    assert outputs == together[:2]
    assert engine.cache.free_pages() == [engine.cache.pools[0].num_pages] and not engine.cache.requests

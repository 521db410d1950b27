"""bin/trace_run against the plain implementation: each request whole; most of it in one step
and the last 32 tokens one by one; in portions of changing size; and mixed with other requests
with so few pages that they are used again. In 32-bit and in bfloat16."""

import numpy as np
import pytest

import plain_gpt2
import replay
from conftest import random_tokens

pytestmark = pytest.mark.gpu


def requests_for(name, config):
    vocab, limit = config["vocab_size"], config["n_positions"]
    lengths = {"A": [5, 17, 33, 100, 128, 64, 65], "B": [1, 9, 40, 64, 63, 33], "C": [130, 257, 600, 40, 191],
               "D": [3, 96, 40, 65, 70], "E": [160, 33, 70, 129, 2]}[name]
    return {f"r{i}": random_tokens(100 + i, min(n, limit), vocab) for i, n in enumerate(lengths)}


MODES = {
    "whole": replay.whole,
    "tail": replay.prefill_then_decode,
    "chunked": replay.chunked,
    "mixed": replay.mixed,
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("mode", list(MODES))
@pytest.mark.parametrize("name", ["A", "B", "C", "D", "E"])
def test_replay_matches_plain(model_dirs, tmp_path, name, mode, dtype):
    folder, config, weights = model_dirs[name]
    requests = requests_for(name, config)
    collector = MODES[mode](requests)
    max_tokens = replay.peak_tokens(collector)  # exactly what is needed: pages are used again
    outputs = replay.run_trace(folder, dtype, collector.steps, tmp_path / "out", max_tokens)
    got = collector.gather(outputs)
    ref = replay.plain_logits(config, weights, requests, bf16=(dtype == "bfloat16"))
    replay.compare(got, ref, **replay.tolerance(dtype))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_replay_hands_out_the_stream_after_every_layer(model_dirs, tmp_path, dtype):
    # --hidden-out: the residual stream after the embedding and after each layer, the rows in the
    # order of the entries, in a mixed trace (whose batches are laid out in another order)
    folder, config, weights = model_dirs["B"]
    requests = requests_for("B", config)
    collector = replay.mixed(requests)
    replay.run_trace(folder, dtype, collector.steps, tmp_path / "out", replay.peak_tokens(collector), hidden_out=tmp_path / "hidden")
    bf16 = dtype == "bfloat16"
    plain = {}
    for name, tokens in requests.items():
        plain[name] = []
        plain_gpt2.forward(config, plain_gpt2.bf16_weights(weights) if bf16 else weights, tokens,
                           stored=plain_gpt2.stored_as_bf16 if bf16 else plain_gpt2._keep, block_outputs=plain[name])
    width, fed = config["n_embd"], {}
    names = ["embedding"] + list(range(config["n_layer"]))
    for step in collector.steps:
        if not step["entries"]:
            continue
        n_rows = sum(len(e["tokens"]) for e in step["entries"])
        for index, name in enumerate(names):
            rows = np.fromfile(tmp_path / "hidden" / f"{step['step']}.{name}.f32", dtype="<f4").reshape(n_rows, width)
            at = 0
            for e in step["entries"]:
                start, n = fed.get(e["id"], 0), len(e["tokens"])
                want = plain[e["id"]][index][start : start + n]
                tol = dict(atol=1e-5, rtol=1e-5) if not bf16 else dict(atol=3e-2, rtol=2e-2)
                np.testing.assert_allclose(rows[at : at + n], want, err_msg=f"step {step['step']} after {name}, request {e['id']}", **tol)
                at += n
        for e in step["entries"]:
            fed[e["id"]] = fed.get(e["id"], 0) + len(e["tokens"])


REAL_SHAPES = {  # two layers at the sizes of the GPT-2 shapes the benchmarks run
    "small": dict(n_embd=768, n_head=12, n_inner=3072),
    "medium": dict(n_embd=1024, n_head=16, n_inner=4096),
    "xl": dict(n_embd=1600, n_head=25, n_inner=6400),
}


@pytest.fixture(scope="module")
def real_shape_dirs(tmp_path_factory):
    """Two layers at a GPT-2 shape's own sizes (small: width 768, 12 heads of 64, inner 3072; xl:
    width 1600, 25 heads, inner 6400; the odd vocabulary of 50,257): the sizes the kernels are tuned
    for, which the tiny models never reach. Made when first asked for."""
    import json

    from conftest import sharpen_attention

    made = {}

    def get(shape):
        if shape not in made:
            config = {"architectures": ["GPT2LMHeadModel"], "model_type": "gpt2", "n_layer": 2, "vocab_size": 50257, "n_positions": 1024,
                      "layer_norm_epsilon": 1e-5, "activation_function": "gelu_new", **REAL_SHAPES[shape]}
            folder = tmp_path_factory.mktemp(f"shape_{shape}")
            weights = plain_gpt2.random_weights(config, 5)
            sharpen_attention(weights, config, factor=3.0)
            (folder / "config.json").write_text(json.dumps(config))
            plain_gpt2.write_safetensors(folder / "model.safetensors", {"transformer." + k: v for k, v in weights.items()})
            made[shape] = (folder, config, weights)
        return made[shape]

    return get


@pytest.fixture
def small_shape_dir(real_shape_dirs):
    return real_shape_dirs("small")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("shape", ["small", "medium"])
def test_replay_at_gpt2_small_and_medium_sizes(real_shape_dirs, tmp_path, dtype, shape):
    # mixed: portions beside decoded tokens of up to four requests, then the last tokens one by one
    # (at small's sizes the bfloat16 decode steps take the layer kernels, at medium's the separate
    # kernels; the portions take the tiled products and the prompt attention; the head runs over the
    # whole odd vocabulary)
    folder, config, weights = real_shape_dirs(shape)
    requests = {f"s{i}": random_tokens(200 + i, n, config["vocab_size"]) for i, n in enumerate((40, 70, 130, 23, 65))}
    collector = replay.mixed(requests, seed=1)
    outputs = replay.run_trace(folder, dtype, collector.steps, tmp_path / "out", replay.peak_tokens(collector))
    ref = replay.plain_logits(config, weights, requests, bf16=(dtype == "bfloat16"))
    replay.compare(collector.gather(outputs), ref, **replay.tolerance(dtype))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_prompts_at_gpt2_small_sizes(small_shape_dir, tmp_path, dtype):
    # two long prompts in one step (the tiled products at hundreds of rows, the prompt attention over
    # several tiles of keys), logits wanted at a few places; then some tokens one by one
    folder, config, weights = small_shape_dir
    requests = {"p": random_tokens(300, 612, config["vocab_size"]), "q": random_tokens(301, 391, config["vocab_size"])}
    collector = replay.Collector()
    head = {name: len(tokens) - 6 for name, tokens in requests.items()}
    collector.add([(name, tokens[: head[name]], sorted({0, 1, 63, 64, 127, 128, 300, head[name] - 1})) for name, tokens in requests.items()])
    for i in range(6):
        collector.add([(name, tokens[head[name] + i : head[name] + i + 1], [0]) for name, tokens in requests.items()],
                      end=list(requests) if i == 5 else [])
    outputs = replay.run_trace(folder, dtype, collector.steps, tmp_path / "out", replay.peak_tokens(collector))
    got = collector.gather(outputs)
    ref = replay.plain_logits(config, weights, requests, bf16=(dtype == "bfloat16"))
    tol = replay.tolerance(dtype)
    for name, rows in got.items():
        assert len(rows) == 8 + 6
        for position, row in rows.items():
            want = ref[name][position]
            err = np.abs(row - want)
            assert (err <= tol["atol"] + tol["rtol"] * np.abs(want)).all(), f"request {name} position {position}: max error {err.max():.3e}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("n_live", [20, 40, 64, 100])
def test_many_decoding_requests_at_gpt2_small_sizes(small_shape_dir, tmp_path, dtype, n_live):
    # decode steps of 20, 40, 64 and 100 rows (beyond the layer kernels: the products of few rows at two
    # and four row tiles, rows handed on in the packed layout, products cut along K; at 100 rows the tiled
    # product on 64 x 64 tiles with finer cuts), after short
    # prompts fed eight requests a step
    folder, config, weights = small_shape_dir
    requests = {f"d{i}": random_tokens(400 + i, 4 + (7 * i) % 23 + 3, config["vocab_size"]) for i in range(n_live)}
    collector = replay.Collector()
    names = list(requests)
    for at in range(0, n_live, 8):
        collector.add([(name, requests[name][:-3], [len(requests[name]) - 4]) for name in names[at : at + 8]])
    for i in range(3, 0, -1):
        collector.add([(name, requests[name][-i : len(requests[name]) - i + 1], [0]) for name in names], end=names if i == 1 else [])
    outputs = replay.run_trace(folder, dtype, collector.steps, tmp_path / "out", replay.peak_tokens(collector))
    got = collector.gather(outputs)
    ref = replay.plain_logits(config, weights, requests, bf16=(dtype == "bfloat16"))
    tol = replay.tolerance(dtype)
    for name, rows in got.items():
        assert len(rows) == 4
        for position, row in rows.items():
            want = ref[name][position]
            err = np.abs(row - want)
            assert (err <= tol["atol"] + tol["rtol"] * np.abs(want)).all(), f"request {name} position {position}: max error {err.max():.3e}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_replay_at_gpt2_xl_sizes(real_shape_dirs, tmp_path, dtype):
    # width 1600 with 25 heads: no layer kernels at this width, other cuts along K, an odd number of heads;
    # a mixed trace, then 40 requests decoding together
    folder, config, weights = real_shape_dirs("xl")
    requests = {f"x{i}": random_tokens(500 + i, n, config["vocab_size"]) for i, n in enumerate((33, 90, 17, 70))}
    collector = replay.mixed(requests, seed=2)
    many = {f"m{i}": random_tokens(600 + i, 5 + (5 * i) % 17, config["vocab_size"]) for i in range(40)}
    names = list(many)
    for at in range(0, 40, 8):
        collector.add([(name, many[name][:-2], [len(many[name]) - 3]) for name in names[at : at + 8]])
    for i in (2, 1):
        collector.add([(name, many[name][-i : len(many[name]) - i + 1], [0]) for name in names], end=names if i == 1 else [])
    outputs = replay.run_trace(folder, dtype, collector.steps, tmp_path / "out", replay.peak_tokens(collector))
    got = collector.gather(outputs)
    assert all(len(rows) == (len(requests[name]) if name in requests else 3) for name, rows in got.items())
    exact = replay.plain_logits(config, weights, {**requests, **many})
    if dtype == "float32":
        tol = replay.tolerance(dtype)
        for name, rows in got.items():
            for position, row in rows.items():
                err = np.abs(row - exact[name][position])
                assert (err <= tol["atol"] + tol["rtol"] * np.abs(exact[name][position])).all(), f"request {name} position {position}: max error {err.max():.3e}"
    else:
        # at this width single logits among millions leave the fixed bound of the tiny models by
        # rounding alone (largest differences 0.02 to 0.034 against 0.025 + 2 %): the bound here is
        # the rounding noise itself
        replay.compare_within_rounding_noise(got, replay.plain_logits(config, weights, {**requests, **many}, bf16=True), exact)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("page_size", [16, 64])
def test_a_context_of_three_thousand_tokens(tmp_path_factory, tmp_path, dtype, page_size):
    # n_positions comes from config.json: a tiny model with 3,100 positions, one request fed in
    # three long portions and then token by token (the prompt attention over dozens of key tiles, the
    # decode attention with sixteen waves over many rounds, block tables of up to 188 pages)
    from conftest import make_plain_model_dir

    config = {"architectures": ["GPT2LMHeadModel"], "model_type": "gpt2", "n_layer": 2, "n_embd": 64, "n_head": 2, "n_inner": 96,
              "vocab_size": 300, "n_positions": 3100, "layer_norm_epsilon": 1e-5, "activation_function": "gelu_new"}
    folder = tmp_path_factory.mktemp("long_context")
    weights = make_plain_model_dir(folder, config, 11)
    tokens = random_tokens(900, 3000, config["vocab_size"])
    collector = replay.Collector()
    at = 0
    for n in (1500, 1000, 492):
        collector.add([("long", tokens[at : at + n], sorted({0, 1, n // 3, n - 2, n - 1}))])
        at += n
    for i in range(at, len(tokens)):
        collector.add([("long", tokens[i : i + 1], [0])], end=["long"] if i == len(tokens) - 1 else [])
    outputs = replay.run_trace(folder, dtype, collector.steps, tmp_path / "out", replay.peak_tokens(collector), page_size=page_size)
    got = collector.gather(outputs)["long"]
    ref = replay.plain_logits(config, weights, {"long": tokens}, bf16=(dtype == "bfloat16"))["long"]
    tol = replay.tolerance(dtype)
    assert len(got) == 15 + 8
    for position, row in got.items():
        err = np.abs(row - ref[position])
        assert (err <= tol["atol"] + tol["rtol"] * np.abs(ref[position])).all(), f"position {position}: max error {err.max():.3e}"


@pytest.mark.parametrize("seed", [3, 4, 5, 6])
def test_other_random_ways_of_mixing_requests(model_dirs, tmp_path, seed):
    # the mixed mode again under other seeds (other portion sizes, other steps a request sits out,
    # other moments at which pages come back and go out again), alternating models and element types
    name, dtype = ("A", "B", "C", "A")[seed - 3], ("float32", "bfloat16")[seed % 2]
    folder, config, weights = model_dirs[name]
    requests = requests_for(name, config)
    collector = replay.mixed(requests, seed=seed, max_live=3 + seed % 2, tail=5 + seed)
    outputs = replay.run_trace(folder, dtype, collector.steps, tmp_path / "out", replay.peak_tokens(collector), page_size=(16, 32, 64, 128)[seed - 3])
    replay.compare(collector.gather(outputs), replay.plain_logits(config, weights, requests, bf16=(dtype == "bfloat16")), **replay.tolerance(dtype))

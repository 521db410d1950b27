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
    lengths = {"A": [5, 17, 33, 100, 128, 64, 65], "B": [1, 9, 40, 64, 63, 33], "C": [130, 257, 600, 40, 191]}[name]
    return {f"r{i}": random_tokens(100 + i, min(n, limit), vocab) for i, n in enumerate(lengths)}


MODES = {
    "whole": replay.whole,
    "tail": replay.prefill_then_decode,
    "chunked": replay.chunked,
    "mixed": replay.mixed,
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("mode", list(MODES))
@pytest.mark.parametrize("name", ["A", "B", "C"])
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


@pytest.fixture(scope="module")
def small_shape_dir(tmp_path_factory):
    """Two layers at GPT-2 small's own sizes (width 768, 12 heads of 64, inner 3072, the odd
    vocabulary of 50,257): the sizes the kernels are tuned for, which the tiny models never reach."""
    import json

    from conftest import sharpen_attention

    config = {"architectures": ["GPT2LMHeadModel"], "model_type": "gpt2", "n_layer": 2, "n_embd": 768, "n_head": 12,
              "n_inner": 3072, "vocab_size": 50257, "n_positions": 1024, "layer_norm_epsilon": 1e-5, "activation_function": "gelu_new"}
    folder = tmp_path_factory.mktemp("small_shape")
    weights = plain_gpt2.random_weights(config, 5)
    sharpen_attention(weights, config, factor=3.0)
    (folder / "config.json").write_text(json.dumps(config))
    plain_gpt2.write_safetensors(folder / "model.safetensors", {"transformer." + k: v for k, v in weights.items()})
    return folder, config, weights


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_replay_at_gpt2_small_sizes(small_shape_dir, tmp_path, dtype):
    # mixed: portions beside decoded tokens of up to four requests, then the last tokens one by one
    # (at these sizes the bfloat16 decode steps take the layer kernels, the portions the tiled
    # products and the prompt attention; the head runs over the whole odd vocabulary)
    folder, config, weights = small_shape_dir
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

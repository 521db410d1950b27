"""bin/trace_run against the plain implementation: each request whole; most of it in one step
and the last 32 tokens one by one; in portions of changing size; and mixed with other requests
with so few pages that they are used again. In 32-bit and in bfloat16."""

import numpy as np
import pytest

import plain_gpt2
import replay
from conftest import random_tokens

pytestmark = pytest.mark.gpu

# float32: the engine's own rounding (sums in another order than numpy's) stays below this.
F32_TOL = dict(atol=2e-5, rtol=1e-4)
# bfloat16 activations between kernels: 8 bits of fraction on values of order one.
BF16_TOL = dict(atol=4e-2, rtol=4e-2)


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
    if dtype == "bfloat16":
        weights = {k: plain_gpt2.round_to_bf16(v) if v.ndim == 2 else v for k, v in weights.items()}
    ref = replay.plain_logits(config, weights, requests)
    replay.compare(got, ref, **(F32_TOL if dtype == "float32" else BF16_TOL))

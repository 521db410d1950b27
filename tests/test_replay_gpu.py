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

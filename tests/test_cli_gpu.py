"""The command line end to end, as a user runs it: a configuration and a seed become a model
folder (python -m mini_llm_amd.cli.random_model), and bin/complete continues a prompt from that
folder. Both run as child processes; the tokens are checked against the plain implementation
(the reference's script is scripts/complete.py:92-129: prompt in, continuation out)."""

import json
import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest

import plain_gpt2
from conftest import TINY_B, TINY_D, random_tokens

pytestmark = pytest.mark.gpu

ROOT = Path(__file__).resolve().parent.parent


def run(command, stdin=None, timeout=300):
    done = subprocess.run([str(c) for c in command], input=stdin, capture_output=True, text=True, timeout=timeout, cwd=ROOT)
    assert done.returncode == 0, f"{command}:\n{done.stdout}\n{done.stderr}"
    return done.stdout


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    """name -> (folder written by the random-weights command, config as a dict, its tensors read
    back by the plain reader)."""
    out = {}
    for name, raw, seed in (("B", TINY_B, 21), ("D", TINY_D, 22)):
        base = tmp_path_factory.mktemp(f"cli_{name}")
        (base / "config.json").write_text(json.dumps(raw))
        printed = run([sys.executable, "-m", "mini_llm_amd.cli.random_model", "--config", base / "config.json", "--seed", seed, "--out", base / "model"])
        assert printed.strip() == str(base / "model")
        config, weights = plain_gpt2.load_model_dir(base / "model")
        # the folder holds the documented draws for this seed
        twin = plain_gpt2.counter_random_weights(raw, seed)
        assert all(np.array_equal(weights[k], twin[k]) for k in twin) and sorted(weights) == sorted(twin)
        out[name] = (base / "model", config, weights)
    return out


def assert_greedy(config, weights, prompt, generated, margin):
    tokens = list(prompt)
    for token in generated:
        logits = plain_gpt2.forward(config, weights, tokens)[-1]
        assert logits[token] >= logits.max() - margin, f"token {token} at length {len(tokens)}"
        tokens.append(token)


@pytest.mark.parametrize("name", ["B", "D"])
def test_complete_continues_a_prompt_greedily(folders, name):
    folder, config, weights = folders[name]
    prompt = random_tokens(40, 9, config["vocab_size"])
    printed = run([ROOT / "bin" / "complete", "--model", folder, "--tokens", ",".join(map(str, prompt)), "--temperature", "0",
                   "--max-new-tokens", "12", "--dtype", "float32"])
    generated = [int(t) for t in printed.strip().split(",")]
    assert len(generated) == 12
    assert_greedy(config, weights, prompt, generated, margin=1e-4)
    assert generated == plain_gpt2.greedy(config, weights, prompt, 12)


def test_complete_cuts_a_long_prompt_from_the_left_and_samples_by_seed(folders):
    folder, config, weights = folders["B"]
    limit = config["n_positions"]                                   # 64
    prompt = random_tokens(41, limit + 10, config["vocab_size"])
    common = [ROOT / "bin" / "complete", "--model", folder, "--tokens", ",".join(map(str, prompt)), "--max-new-tokens", "6", "--dtype", "float32"]
    greedy = [int(t) for t in run(common + ["--temperature", "0"]).strip().split(",")]
    kept = prompt[-(limit - 6):]                                     # room for the new tokens (scripts/complete.py:92-110)
    assert greedy == plain_gpt2.greedy(config, weights, kept, 6)
    # a temperature samples; the seed decides
    a = run(common + ["--temperature", "1.2", "--top-p", "0.9", "--seed", "5"])
    b = run(common + ["--temperature", "1.2", "--top-p", "0.9", "--seed", "5"])
    c = run(common + ["--temperature", "1.2", "--top-p", "0.9", "--seed", "6"])
    assert a == b and len(a.strip().split(",")) == 6 and (a != c or a != run(common + ["--temperature", "1.2", "--top-p", "0.9", "--seed", "7"]))


def test_the_prompt_loop(folders):
    folder, config, weights = folders["B"]
    prompt = random_tokens(42, 5, config["vocab_size"])
    line = " ".join(map(str, prompt))
    printed = run([ROOT / "bin" / "complete", "--model", folder, "--temperature", "0", "--max-new-tokens", "4", "--dtype", "bfloat16"],
                  stdin=f"{line}\n/history\n/clear\n/history\nnot numbers\n/exit\n").strip().splitlines()
    generated = [int(t) for t in printed[0].split("> ")[-1].split()]
    assert len(generated) == 4
    assert_greedy(config, plain_gpt2.bf16_weights(weights), prompt, generated, margin=0.05)
    # /history shows the turn once; after /clear nothing
    shown = [l for l in printed if " ".join(map(str, generated)) in l]
    assert len(shown) == 2

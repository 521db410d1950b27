"""Helpers for the replay tests: traces in the four ways of cutting the work, a driver for
bin/trace_run, and the plain implementation's logits to compare with."""

import json
import subprocess
import sys
from pathlib import Path

import numpy as np

import plain_gpt2

ROOT = Path(__file__).resolve().parent.parent

# float32: the engine's own rounding (sums in another order than numpy's) is a few 1e-7 at 128
# positions and 7e-6 at 600 with sharp attention; the bound leaves a factor of three.
F32_TOL = dict(atol=2e-5, rtol=2e-5)
# bfloat16, against the plain implementation storing the same tensors in bfloat16: what is left is
# single roundings that fall the other way (sums in another order) and what the softmax makes of
# them; measured 2e-3 to 1.6e-2 on logits up to 2.4.
BF16_TOL = dict(atol=2.5e-2, rtol=2e-2)


def tolerance(dtype: str) -> dict:
    return F32_TOL if dtype == "float32" else BF16_TOL


def run_trace(model_dir, dtype, steps, out_dir, max_tokens, page_size=None, timeout=600, hidden_out=None):
    """Runs bin/trace_run over the steps; returns {step: array [wanted, vocab]}."""
    out_dir = Path(out_dir)
    cmd = [sys.executable, str(ROOT / "bin" / "trace_run"), "--model", str(model_dir), "--dtype", dtype,
           "--out", str(out_dir), "--max-tokens", str(max_tokens)]
    if page_size:
        cmd += ["--page-size", str(page_size)]
    if hidden_out:
        cmd += ["--hidden-out", str(hidden_out)]
    text = "".join(json.dumps(s) + "\n" for s in steps)
    done = subprocess.run(cmd, input=text, capture_output=True, text=True, timeout=timeout)
    assert done.returncode == 0, f"trace_run failed ({done.returncode}):\n{done.stderr[-3000:]}"
    assert [l for l in done.stdout.split("\n") if l.startswith("done")] == [f"done {s['step']}" for s in steps]
    vocab = json.loads((Path(model_dir) / "config.json").read_text())["vocab_size"]
    out = {}
    for s in steps:
        wanted = sum(len(e.get("want", [])) for e in s["entries"])
        path = out_dir / f"{s['step']}.f32"
        if wanted:
            out[s["step"]] = np.fromfile(path, dtype="<f4").reshape(wanted, vocab)
        else:
            assert not path.exists()
    return out


class Collector:
    """Gathers, per request, the logits of each position from the steps' outputs."""

    def __init__(self):
        self.steps = []
        self.where = []  # per step: list of (request, position) in output order
        self.fed = {}

    def add(self, entries, end=()):
        """entries: [(request, tokens, want)]; positions follow from what was fed before."""
        places, recs = [], []
        for request, tokens, want in entries:
            start = self.fed.get(request, 0)
            recs.append({"id": request, "tokens": [int(t) for t in tokens], "want": [int(w) for w in want]})
            places += [(request, start + w) for w in want]
            self.fed[request] = start + len(tokens)
        self.steps.append({"step": len(self.steps), "entries": recs, "end": list(end)})
        self.where.append(places)
        for request in end:
            self.fed.pop(request, None)

    def gather(self, outputs):
        """{request: {position: logits row}}"""
        got = {}
        for step, places in zip(self.steps, self.where):
            if places:
                rows = outputs[step["step"]]
                for row, (request, position) in zip(rows, places):
                    got.setdefault(request, {})[position] = row
        return got


def whole(requests):
    """Each request alone, all its tokens in one step, every position wanted."""
    c = Collector()
    for name, tokens in requests.items():
        c.add([(name, tokens, range(len(tokens)))], end=[name])
    return c


def prefill_then_decode(requests, tail=32):
    """All but the last ``tail`` tokens in one step, then the rest one by one."""
    c = Collector()
    for name, tokens in requests.items():
        head = max(1, len(tokens) - tail)
        c.add([(name, tokens[:head], range(head))])
        for i in range(head, len(tokens)):
            c.add([(name, tokens[i : i + 1], [0])], end=[name] if i == len(tokens) - 1 else [])
        if head == len(tokens):
            c.add([], end=[name])
    return c


def chunked(requests, sizes=(7, 2, 16, 3, 2, 33, 5, 2, 64, 11)):
    """Portions of changing size, down to two tokens."""
    c = Collector()
    for name, tokens in requests.items():
        at, i = 0, 0
        while at < len(tokens):
            n = min(sizes[i % len(sizes)], len(tokens) - at)
            i += 1
            last = at + n == len(tokens)
            c.add([(name, tokens[at : at + n], range(n))], end=[name] if last else [])
            at += n
    return c


def mixed(requests, seed=0, max_live=4, tail=12):
    """Up to ``max_live`` live requests: portions of some beside single decoded tokens of
    others; a request is sometimes left out of a step; requests join as others end."""
    rng = np.random.default_rng(seed)
    c = Collector()
    waiting = list(requests.items())
    live = {}  # name -> [tokens, fed]
    while waiting or live:
        while waiting and len(live) < max_live:
            name, tokens = waiting.pop(0)
            live[name] = [tokens, 0]
        entries, ended = [], []
        for name, (tokens, fed) in list(live.items()):
            if len(live) > 1 and rng.random() < 0.2:
                continue  # left out of this step
            left = len(tokens) - fed
            if left <= tail:
                n = 1  # the last tokens go one by one, as decoded tokens would
            else:
                n = int(min(left - tail, rng.choice([2, 3, 5, 8, 13, 21, 40])))
            entries.append((name, tokens[fed : fed + n], range(n)))
            live[name][1] = fed + n
            if fed + n == len(tokens):
                ended.append(name)
                del live[name]
        if entries:
            c.add(entries, end=ended)
    return c


def peak_tokens(collector, page=64):
    """The most tokens live requests hold at any time, each rounded up to a multiple of ``page``."""
    held, peak = {}, 0
    for step in collector.steps:
        for e in step["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        peak = max(peak, sum(-(-n // page) * page for n in held.values()))
        for name in step["end"]:
            held.pop(name, None)
    return peak


def plain_logits(config, weights, requests, dtype=np.float64, bf16=False):
    """The plain implementation's logits; ``bf16``: as a bfloat16 run stores tensors (matrices,
    tables and the activations between kernels rounded to bfloat16, arithmetic in float64)."""
    if bf16:
        weights = plain_gpt2.bf16_weights(weights)
    stored = plain_gpt2.stored_as_bf16 if bf16 else plain_gpt2._keep
    return {name: plain_gpt2.forward(config, weights, tokens, dtype, stored) for name, tokens in requests.items()}


def compare(got, ref, atol, rtol):
    """Every position of every request; on a mismatch names the first wrong place."""
    for name, rows in ref.items():
        assert set(got[name]) == set(range(len(rows))), f"{name}: positions {sorted(set(range(len(rows))) - set(got[name]))} missing"
        for position in range(len(rows)):
            a, b = got[name][position].astype(np.float64), rows[position]
            err = np.abs(a - b)
            bad = err > atol + rtol * np.abs(b)
            assert not bad.any(), (
                f"request {name!r} position {position}: {int(bad.sum())} logits differ, max error {err.max():.3e} "
                f"(allowed {atol:g} + {rtol:g}*|ref|); first wrong position of this request"
            )


def compare_within_rounding_noise(got, ref_rounded, ref_exact, max_share=1.0, rms_share=0.6):
    """For bfloat16 at widths where a fixed bound no longer fits (rounding noise grows with the
    width and the depth): the engine may differ from the plain implementation that stores the same
    tensors in bfloat16 by less than that implementation itself differs from exact arithmetic. Per
    request: at every position the largest difference stays under ``max_share`` of the largest
    difference between the rounded and the exact plain logits of that request, and the root mean
    square under ``rms_share`` of theirs. Measured at width 1,600: 0.3 to 0.4 of either (most
    roundings fall the same way in both); a wrong key, row or page gives differences of the size
    of the logits, tens of times the noise."""
    for name, rows in got.items():
        exact, rounded = ref_exact[name], ref_rounded[name]
        noise = np.abs(rounded - exact)
        noise_max, noise_rms = noise.max(), np.sqrt((noise**2).mean())
        squares, count = 0.0, 0
        for position, row in sorted(rows.items()):
            err = np.abs(row.astype(np.float64) - rounded[position])
            assert err.max() <= max_share * noise_max, (
                f"request {name!r} position {position}: max error {err.max():.3e}, the rounding noise of this request is {noise_max:.3e}")
            squares += float((err**2).sum())
            count += err.size
        rms = np.sqrt(squares / count)
        assert rms <= rms_share * noise_rms, f"request {name!r}: rms error {rms:.3e}, the rounding noise has {noise_rms:.3e}"

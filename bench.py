"""Decode and prefill throughput of the engine on one MI355X, GPT-2 small with random weights.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--dtype bfloat16|float32] [--batch 8]

A step is one decode step: every live sequence gets one new token (greedy, sampled on the
device and fed back). Sequences start from 512-token uniform-random prompts and decode towards
1,024 tokens; when they are full they are given back and prefilled again outside the timed
region, so that exactly K steps are timed. Before anything is timed, 8 decoded tokens are compared
with a whole-prompt step and with the plain implementation under tests/ (--no-check skips that).
Prints one JSON line: the headline in bfloat16, the same figures in 32-bit under "points_fp32", and
under "kernels" what the kernels a step's time goes to reach of their own roofline. The reference's
counterpart is engine/bench/bench_batch.c (batched decode at a context) and engine/bench/bench.c."""

from __future__ import annotations

import argparse
import json
import sys
import time
from pathlib import Path

sys.path.insert(0, str(Path(__file__).resolve().parent))

# MI355X's published peaks
HBM_GBS = 8000.0
PEAK_FLOPS = {"bfloat16": 2.5e15, "float32": 157.3e12}

SMALL = {"architectures": ["GPT2LMHeadModel"], "n_layer": 12, "n_embd": 768, "n_head": 12, "n_inner": 3072,
         "vocab_size": 50257, "n_positions": 1024, "layer_norm_epsilon": 1e-5, "activation_function": "gelu_new"}
PROMPT_LEN, CONTEXT, SEED = 512, 1024, 5


def element_size(dtype: str) -> int:
    return 2 if dtype == "bfloat16" else 4


def matrix_elements(c) -> int:
    per_layer = c.n_embd * 3 * c.n_embd + c.n_embd * c.n_embd + 2 * c.n_embd * c.n_inner
    return c.n_layer * per_layer


def decode_bytes(c, dtype: str, context_lens) -> float:
    """What a decode step has to read: every weight it uses once, and the live requests' cache."""
    e = element_size(dtype)
    weights = (matrix_elements(c) + c.vocab_size * c.n_embd) * e          # matrices and the tied head
    vectors = c.n_layer * (9 * c.n_embd + c.n_inner) * 4 + 2 * c.n_embd * 4   # biases and norms, 32-bit
    cache = sum(context_lens) * 2 * c.n_embd * c.n_layer * e
    return float(weights + vectors + cache)


def prefill_flops(c, lengths, wanted_rows: int) -> float:
    tokens = sum(lengths)
    linear = 2.0 * tokens * matrix_elements(c)
    attention = sum(2.0 * 2.0 * (n * (n + 1) / 2) * c.n_embd * c.n_layer for n in lengths)  # QK^T and PV, causal
    head = 2.0 * wanted_rows * c.vocab_size * c.n_embd
    return linear + attention + head


class DecodeBench:
    def __init__(self, engine, batch: int, prompt_len: int = PROMPT_LEN):
        import numpy as np

        self.engine, self.batch, self.prompt_len = engine, batch, prompt_len
        rng = np.random.default_rng(SEED + 1)
        self.prompts = [rng.integers(0, engine.config.vocab_size, prompt_len).tolist() for _ in range(batch)]
        self.handles, self.last, self.length = [], [], 0

    def start(self):
        """Takes the sequences and prefills their prompts (a few at a time, untimed)."""
        from mini_llm_amd.engine import StepEntry
        from mini_llm_amd.sampling import SamplingParams

        self.stop()
        self.handles = [self.engine.try_take_cache() for _ in range(self.batch)]
        self.last = []
        for i in range(0, self.batch, 4):
            entries = [StepEntry(h, p, [self.prompt_len - 1]) for h, p in zip(self.handles[i : i + 4], self.prompts[i : i + 4])]
            logits = self.engine.runner.step(entries)
            self.last += self.engine.sampler.sample(logits, [SamplingParams()] * len(entries), [0] * len(entries)).cpu().tolist()
        self.length = self.prompt_len

    def stop(self):
        for handle in self.handles:
            self.engine.release_cache(handle)
        self.handles = []

    def run(self, steps: int, warmup: int):
        """(seconds, bytes a step had to read on average) over exactly ``steps`` timed steps."""
        import torch

        self.start()
        for _ in range(warmup):
            if self.length >= CONTEXT:
                self.start()
            self.last = self.engine.decode_batch(self.handles, self.last)
            self.length += 1
        seconds, bytes_read, done = 0.0, 0.0, 0
        config, dtype = self.engine.config, self.engine.options.dtype
        while done < steps:
            if self.length >= CONTEXT - 1:
                # new sequences: one untimed step from the host's tokens leaves every sequence's newest token on the
                # device, where the queued steps below take it from
                self.start()
                self.last = self.engine.decode_batch(self.handles, self.last)
                self.length += 1
            n = min(steps - done, CONTEXT - self.length)
            torch.cuda.synchronize()
            begin = time.perf_counter()
            # Queued decoding, one step ahead: step k+1 takes its tokens from the device, where
            # step k's sampler left them, and is launched before the host reads step k's tokens.
            self.engine.decode_batch_enqueue(self.handles)
            for _ in range(n - 1):
                self.engine.decode_batch_enqueue(self.handles)
                self.last = self.engine.take()
            self.last = self.engine.take()
            torch.cuda.synchronize()
            seconds += time.perf_counter() - begin
            for k in range(n):
                bytes_read += decode_bytes(config, dtype, [self.length + k + 1] * self.batch)
            self.length += n
            done += n
        self.stop()
        return seconds, bytes_read / steps


def measure_prefill(engine, runs: int = 5):
    import numpy as np
    import torch

    from mini_llm_amd.engine import StepEntry

    rng = np.random.default_rng(SEED + 2)
    lengths = [CONTEXT, CONTEXT]
    # token ids as int32 arrays, as a front end that has tokenised the prompts holds them (a list of Python integers
    # would be turned into one first, 25 us a thousand tokens)
    prompts = [rng.integers(0, engine.config.vocab_size, n).astype(np.int32) for n in lengths]
    times = []
    # a shape of step that keeps coming is replayed from a captured graph; the warm-up runs go past the capture
    warm = 2 + max(0, engine.runner.portion_graph_after if engine.runner.use_graphs else 0)
    replayed_before = engine.runner.portion_graph_steps
    for _ in range(runs + warm):
        handles = [engine.try_take_cache() for _ in prompts]
        entries = [StepEntry(h, p, [len(p) - 1]) for h, p in zip(handles, prompts)]
        torch.cuda.synchronize()
        begin = time.perf_counter()
        engine.runner.step(entries)
        torch.cuda.synchronize()
        times.append(time.perf_counter() - begin)
        for h in handles:
            engine.release_cache(h)
    seconds = float(np.median(times[warm:]))
    tokens = sum(lengths)
    flops = prefill_flops(engine.config, lengths, len(prompts))
    return {"value": round(tokens / seconds, 1), "tokens": tokens, "ms": round(seconds * 1e3, 3),
            "frac": round(flops / seconds / PEAK_FLOPS[engine.options.dtype], 4), "from_graph": engine.runner.portion_graph_steps - replayed_before >= runs}


def kernel_times_inside_a_step(engine, make_entries, choose: bool, reps: int = 5):   # (reps_of_a_step: what callers plan room for)
    """(names, microseconds): the kernels of one real step of the engine, in order, and what each takes INSIDE the step.

    The step goes through the engine's own step function and is captured as generation captures it. It is captured once
    for every n with only its first n kernels really launched (ops.library.first_launches), and the replay of each such
    graph is timed: kernel n's time is the difference between two of them. So a time holds what the kernel costs where it
    stands: its start behind the kernel before it, and its first trip to memory for what that one wrote. (The first
    kernel's figure also holds what a replay and the two events around it cost by themselves.) ``make_entries()`` opens the step's requests and returns
    (entries, handles); they are given back after each capture."""
    import numpy as np
    import torch

    import ctypes

    from mini_llm_amd.engine.step import ModelRunner
    from mini_llm_amd.ops.library import check, first_launches, library

    model, cache, device = engine.model, engine.cache, engine.options.device

    def captured(limit, period=None):
        runner = ModelRunner(model, cache, device, portion_graph_after=1, lanes_from=engine.runner.lanes_from)
        entries, handles = make_entries()
        with first_launches(limit, period) as seen:
            runner.step(entries, choose=choose)
        graphs = list(runner._graphs.values()) + list(runner._portion_graphs.values())
        assert len(graphs) == 1 and graphs[0].graph is not None, "the step was not captured"
        # the eager run before the capture and the capture itself ask for the same launches
        names = seen.asked[: len(seen.asked) // 2]
        assert names == seen.asked[len(names):], "the captured step is not the step that ran"
        return runner, graphs[0].graph, names, handles

    # Between two timed replays the caches are emptied by a read of 512 MiB of other memory: in generation a step's weights and
    # cache rows have been pushed out by the rest of the step before they are read again, but a short graph replayed by
    # itself would find everything still in the 256 MB memory-side cache.
    lib = library()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    other = torch.zeros((512 << 20) // 4, dtype=torch.float32, device=device)
    sink = torch.zeros(1, dtype=torch.float32, device=device)

    def replay_us(graph):
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        graph.replay()
        samples = []
        for _ in range(reps):
            check(lib.mllm_probe_read(ctypes.c_void_p(other.data_ptr()), other.numel() * 4, ctypes.c_void_p(sink.data_ptr()), 2048, stream))
            start.record()
            graph.replay()
            stop.record()
            torch.cuda.synchronize()
            samples.append(start.elapsed_time(stop) * 1e3)
        return float(np.median(samples))

    def forget(runner, handles):
        runner.drop_graphs()
        for h in handles:
            engine.release_cache(h)

    runner, graph, names, handles = captured(None)   # for the names and their number
    forget(runner, handles)
    upto = []
    for n in range(1, len(names) + 1):
        runner, graph, _, handles = captured(n, len(names))   # the step runs once before its capture: the first n of each run
        upto.append(replay_us(graph))
        forget(runner, handles)
    each = [upto[0]] + [max(0.0, upto[i] - upto[i - 1]) for i in range(1, len(upto))]
    return names, each


def reps_of_a_step() -> int:
    return 5


def measure_kernels(engine, batch: int = 8, context: int = 776, decode: bool = True):
    """What the kernels that a step's time goes to take inside the step and reach of their own roofline
    (``kernel_times_inside_a_step``): for a 2,048-token prompt step the four products of a layer and the prompt
    attention (flops / time / the matrix cores' peak), for a greedy decode step of ``batch`` sequences at ``context``
    tokens the kernels of a layer, the head and the choice of the tokens (the bytes each has to read / time / the
    memory's peak); a layer's kernel is the mean over the layers. The reference prices its kernels against a pure read
    of the same bytes (docs/kernels/010_matvec_batch.md:20,108-117) and times the stages of its steps with event pairs
    (engine/src/gpu_timer.cu:13-120)."""
    import numpy as np

    from mini_llm_amd.engine import StepEntry

    config, dtype = engine.config, engine.options.dtype
    e = element_size(dtype)
    d, ff, n_layer, vocab = config.n_embd, config.n_inner, config.n_layer, config.vocab_size
    rng = np.random.default_rng(SEED + 4)
    out = {}

    def note(name, us, work, peak, unit):
        out[name] = {"us": round(us, 2), "frac": round(work / (us * 1e-6) / peak, 4) if us > 0 else None, "of": unit}

    def by_layer(names, each, tail):
        """The step's kernels as (first, [per layer: the mean over the layers of each kernel of a layer], last ``tail``), if
        the kernels between the first and the last ones fall into n_layer equal runs; else None."""
        middle = len(names) - 1 - tail
        if middle <= 0 or middle % n_layer:
            return None
        per = middle // n_layer
        layers = [(names[1 + k], float(np.mean([each[1 + layer * per + k] for layer in range(n_layer)]))) for k in range(per)]
        return (names[0], each[0]), layers, list(zip(names[-tail:], each[-tail:]))

    # --- a prompt step of two 1,024-token prompts
    lengths = [CONTEXT, CONTEXT]
    prompts = [rng.integers(0, vocab, n).astype(np.int32) for n in lengths]

    def prompt_step():
        handles = [engine.try_take_cache() for _ in lengths]
        return [StepEntry(h, p, [len(p) - 1]) for h, p in zip(handles, prompts)], handles

    names, each = kernel_times_inside_a_step(engine, prompt_step, choose=False)
    rows = sum(lengths)
    peak, unit = PEAK_FLOPS[dtype], f"{'bf16' if dtype == 'bfloat16' else 'fp32'} matrix peak"
    cut = by_layer(names, each, tail=2)   # the final norm and the head
    out["prefill_step"] = {"us": round(sum(each), 1), "kernels": len(names)}
    if cut is not None and len(cut[1]) == 7:
        (_, norm_1), (_, qkv), (_, attention), (_, proj), (_, norm_2), (_, up), (_, down) = cut[1]
        note("prefill_qkv_product", qkv, 2.0 * rows * d * 3 * d, peak, unit)
        note("prefill_attention", attention, sum(4.0 * (n * (n + 1) / 2) * d for n in lengths), peak, unit)
        note("prefill_out_product", proj, 2.0 * rows * d * d, peak, unit)
        note("prefill_up_product", up, 2.0 * rows * d * ff, peak, unit)
        note("prefill_down_product", down, 2.0 * rows * d * ff, peak, unit)
        out["prefill_norms"] = {"us": round(norm_1 + norm_2, 2)}
    else:
        out["prefill_step"]["by_entry_point"] = _by_entry_point(names, each)
    if not decode:
        return out

    # --- a greedy decode step: ``batch`` sequences that hold ``context`` tokens each (the replays of the whole step move
    # the sequences on by a token each, and must stay on the page the step has reserved)
    page = engine.cache.page_size
    assert page - context % page > reps_of_a_step() + 8, "the decode step's replays need room on the sequences' newest page"
    stored = [rng.integers(0, vocab, context).tolist() for _ in range(batch)]

    def decode_step():
        handles = [engine.try_take_cache() for _ in range(batch)]
        for i in range(0, batch, 4):
            engine.runner.step([StepEntry(h, tokens, []) for h, tokens in zip(handles[i : i + 4], stored[i : i + 4])])
        return [StepEntry(h, [int(rng.integers(0, vocab))], [0]) for h in handles], handles

    names, each = kernel_times_inside_a_step(engine, decode_step, choose=True)
    hbm = HBM_GBS * 1e9
    out["decode_step"] = {"us": round(sum(each), 1), "kernels": len(names)}
    cut = by_layer(names, each, tail=3)   # the final norm, the head and the choice
    cache_bytes = batch * context * 2.0 * d * e
    if cut is not None and [name for name, _ in cut[1]] == ["decode_attention_half", "decode_mlp_half"]:
        note("decode_attention_half", cut[1][0][1], 4.0 * d * d * e + cache_bytes, hbm, "HBM peak")
        note("decode_mlp_half", cut[1][1][1], 2.0 * d * ff * e, hbm, "HBM peak")
    elif cut is not None:
        layer_us = sum(us for _, us in cut[1])
        note("decode_layer", layer_us, (4.0 * d * d + 2.0 * d * ff) * e + cache_bytes, hbm, "HBM peak")
        out["decode_layer"]["by_entry_point"] = _by_entry_point([name for name, _ in cut[1]], [us for _, us in cut[1]])
    if cut is not None:
        out["decode_embed"] = {"us": round(cut[0][1], 2), "holds": "what a replay costs by itself"}
        (_, final_norm), (_, head), (_, choice) = cut[2]
        out["decode_final_norm"] = {"us": round(final_norm, 2)}
        note("decode_head", head, float(vocab) * d * e, hbm, "HBM peak")
        out["decode_choice"] = {"us": round(choice, 2)}
    else:
        out["decode_step"]["by_entry_point"] = _by_entry_point(names, each)
    return out


def _by_entry_point(names, each):
    """entry point -> [launches, microseconds in sum], for a step whose kernels do not fall into the pattern looked for."""
    table = {}
    for name, us in zip(names, each):
        entry = table.setdefault(name, [0, 0.0])
        entry[0] += 1
        entry[1] = round(entry[1] + us, 2)
    return table


def check_before_timing(engine, host_weights=None, n_new: int = 8):
    """The gate before anything is timed, as the reference's bench has one (engine/bench/bench.c:30-31,
    92-113: its GPU against its CPU path on 8 tokens, scaled difference <= 1e-3 and the same next
    token). Two sequences are decoded greedily for 8 tokens the way the timed steps run (single
    tokens over the cache, replayed from a graph). Then (1) each whole sequence runs again as one
    prompt step, through the other kernels (tiled products, prompt attention), and (2) with
    ``host_weights`` (the model's tensors as numpy arrays) the first sequence runs through the plain
    implementation under tests/ (numpy, float64, no cache; storing in bfloat16 what a bfloat16 run
    stores): the logits at the decoded places must agree with both. Returns the largest
    difference / largest logit of (1) and of (2)."""
    import numpy as np
    import torch

    from mini_llm_amd.engine import StepEntry

    rng = np.random.default_rng(SEED + 3)
    prompts = [rng.integers(0, engine.config.vocab_size, n).tolist() for n in (40, 70)]
    handles = [engine.try_take_cache() for _ in prompts]
    logits = engine.runner.step([StepEntry(h, p, [len(p) - 1]) for h, p in zip(handles, prompts)])
    stepwise, sequences = [[] for _ in prompts], [list(p) for p in prompts]
    for _ in range(n_new):
        rows = logits.float().cpu().numpy()
        for i, row in enumerate(rows):
            stepwise[i].append(row)
            sequences[i].append(int(row.argmax()))
        logits = engine.runner.step([StepEntry(h, [seq[-1]], [0]) for h, seq in zip(handles, sequences)])
    for h in handles:
        engine.release_cache(h)
    bf16 = engine.options.dtype == "bfloat16"

    def compare(what, got_rows, want_rows, limit, sequence):
        worst = 0.0
        for k, (a, b) in enumerate(zip(got_rows, want_rows)):
            scaled = float(np.abs(a - b).max() / np.abs(b).max())
            worst = max(worst, scaled)
            top = np.sort(b)[-2:]
            clear = (top[1] - top[0]) > 2 * limit * np.abs(b).max()   # a near tie may fall either way
            if not scaled <= limit or (clear and int(a.argmax()) != int(b.argmax())):
                raise SystemExit(f"bench.py: decoding and {what} disagree at sequence {sequence}, new token {k}: scaled difference "
                                 f"{scaled:.3e} (allowed {limit:g}), next token {int(a.argmax())} vs {int(b.argmax())}; nothing was timed")
        return worst

    worst_whole = 0.0
    limit = 5e-2 if bf16 else 1e-3   # bfloat16 rounds every stored activation to 3 digits, and the two paths round at different places
    for i, (prompt, seq) in enumerate(zip(prompts, sequences)):
        handle = engine.try_take_cache()
        fed = seq[:-1]
        whole = engine.runner.step([StepEntry(handle, fed, list(range(len(prompt) - 1, len(fed))))]).float().cpu().numpy()
        engine.release_cache(handle)
        worst_whole = max(worst_whole, compare("the whole-prompt step", stepwise[i], whole, limit, i))
    torch.cuda.synchronize()
    worst_plain = None
    if host_weights is not None:
        sys.path.insert(0, str(Path(__file__).resolve().parent / "tests"))
        import plain_gpt2

        raw = engine.config.to_dict()
        weights = plain_gpt2.bf16_weights(host_weights) if bf16 else host_weights
        fed = sequences[0][:-1]
        plain = plain_gpt2.forward(raw, weights, fed, stored=plain_gpt2.stored_as_bf16 if bf16 else plain_gpt2._keep)
        # against exact arithmetic over the same stored numbers: 2e-2 of the largest logit in bfloat16 (observed: a few 1e-3)
        worst_plain = compare("the plain implementation", stepwise[0], plain[len(prompts[0]) - 1 :], 2e-2 if bf16 else 1e-3, 0)
    return worst_whole, worst_plain


MEDIUM = dict(SMALL, n_layer=24, n_embd=1024, n_head=16, n_inner=4096)
XL = dict(SMALL, n_layer=48, n_embd=1600, n_head=25, n_inner=6400)
SHAPES = {"small": (SMALL, SEED), "medium": (MEDIUM, 6), "xl": (XL, 7)}  # the shapes and weight seeds the baseline names


def measure_serving(dtype: str, temperature: float, step_ahead: bool = True):
    """Continuous batching through the scheduler: 64 concurrent requests on the GPT-2 medium shape,
    prompts of 32 to 768 uniform-random ids, 256 new tokens each, prompts cut into portions under a
    budget of 512 tokens a step and run beside the decodes."""
    import numpy as np
    import torch

    from mini_llm_amd.config import config_from_dict
    from mini_llm_amd.engine.engine import Engine, EngineOptions
    from mini_llm_amd.engine.scheduler import Request
    from mini_llm_amd.sampling import SamplingParams

    config = config_from_dict(MEDIUM)
    engine = Engine.from_random(config, 6, EngineOptions(dtype=dtype, max_sessions=64, max_tokens=64 * CONTEXT, max_tokens_per_step=512,
                                                        step_ahead=step_ahead))
    rng = np.random.default_rng(6)
    prompts = [rng.integers(0, config.vocab_size, int(n)).tolist() for n in rng.integers(32, 769, 64)]
    counts = [0] * len(prompts)

    def run_once():
        for i, prompt in enumerate(prompts):
            def emit(token, finish, i=i):
                counts[i] += 1
            engine.submit(Request(prompt, on_token=emit, on_error=lambda message: None, max_new_tokens=256,
                                  sampling=SamplingParams(temperature=temperature, seed=i)))
        torch.cuda.synchronize()
        begin = time.perf_counter()
        engine.scheduler.run_until_idle()
        torch.cuda.synchronize()
        return time.perf_counter() - begin

    for _ in range(4):   # warm-up: the decode steps are captured in the first run, the padded shapes of the mixed steps at their fourth coming
        run_once()
    for i in range(len(counts)):
        counts[i] = 0
    before = engine.stats()
    seconds = run_once()
    after = engine.stats()
    generated, prompt_tokens = sum(counts), sum(len(p) for p in prompts)
    return {"model": "gpt2-medium shape", "dtype": dtype, "requests": len(prompts), "prompt_tokens": prompt_tokens,
            "generated_tokens": generated, "seconds": round(seconds, 3), "generated_tokens_per_s": round(generated / seconds, 1),
            "all_tokens_per_s": round((generated + prompt_tokens) / seconds, 1), "steps": after["steps"] - before["steps"],
            "temperature": temperature, "preemptions": after["preemptions"] - before["preemptions"],
            "step_ahead": step_ahead}


def measure_peaks():
    """What this machine reaches with nothing in the way: a pure read of 1 GiB, and the matrix
    cores with operands in registers (the library's two probes)."""
    import ctypes

    import torch

    from mini_llm_amd.ops.library import check, library

    lib = library()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    n_bytes = 1 << 30
    buffer = torch.zeros(n_bytes // 4, dtype=torch.float32, device="cuda:0")
    blocks, iterations = 2048, 20000
    out = torch.zeros(blocks * 256, dtype=torch.float32, device="cuda:0")

    def timed(fn, reps=3):
        fn()
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        best = float("inf")
        for _ in range(reps):
            start.record()
            fn()
            stop.record()
            torch.cuda.synchronize()
            best = min(best, start.elapsed_time(stop) / 1e3)
        return best

    read_s = timed(lambda: check(lib.mllm_probe_read(ctypes.c_void_p(buffer.data_ptr()), n_bytes, ctypes.c_void_p(out.data_ptr()), 4096, stream)))
    result = {"hbm_read_GBs": round(n_bytes / read_s / 1e9, 1)}
    for name, code, flops in (("bf16", 1, 32768.0), ("fp32", 0, 4096.0)):
        s = timed(lambda: check(lib.mllm_probe_mfma(ctypes.c_void_p(out.data_ptr()), blocks, iterations, code, stream)))
        result[f"mfma_{name}_TFLOPs"] = round(blocks * 4 * iterations * 4 * flops / s / 1e12, 1)
    return result


def emit(record: dict, path) -> None:
    line = json.dumps(record)
    print(line)
    if path:
        Path(path).write_text(line + "\n")


def main() -> int:
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=256)
    parser.add_argument("--warmup", type=int, default=16)
    parser.add_argument("--dtype", default="bfloat16", choices=("bfloat16", "float32"))
    parser.add_argument("--batch", type=int, default=8)
    parser.add_argument("--lanes-from", type=int, default=None, help="decode steps of at least so many sequences run two halves side by side (0: never; default: the engine's)")
    parser.add_argument("--shape", default="small", choices=("small", "medium", "xl"), help="the GPT-2 shape that is run (the headline is small)")
    parser.add_argument("--prompt-len", "--prompt-tokens", dest="prompt_len", type=int, default=PROMPT_LEN,
                        help="tokens of each sequence's prompt before decoding is timed (--prompt-tokens is the reference's name: engine/bench/bench_options.c:25-94)")
    parser.add_argument("--context", type=int, default=CONTEXT, help="the model's positions: sequences decode towards this length, and the prompt step is two prompts of this length "
                        "(the headline is 1024; a longer one runs the same layer sizes with a longer position table)")
    parser.add_argument("--json", default=None, metavar="PATH", help="also write the printed record to this file (the reference's option)")
    parser.add_argument("--layers", type=int, default=None, help="run fewer layers than the configuration has (both numbers are reported)")
    parser.add_argument("--no-check", action="store_true", help="skip the comparison of decoding with a whole-prompt step before timing")
    parser.add_argument("--no-points", action="store_true", help="skip the batch 1 / batch 64 points, the prefill, the kernels and the other precision")
    parser.add_argument("--one-dtype", action="store_true", help="skip the figures in the other precision")
    parser.add_argument("--no-kernels", action="store_true", help="with --prefill-only: without the times of the step's kernels (for profiling: those take thousands of launches of their own)")
    parser.add_argument("--prefill-only", action="store_true", help="run the 2,048-token prefill alone (for profiling) and print its record")
    parser.add_argument("--serving", action="store_true", help="continuous batching of 64 requests on the GPT-2 medium shape through the scheduler")
    parser.add_argument("--temperature", type=float, default=0.0, help="sampling temperature of --serving (0: greedy)")
    parser.add_argument("--step-by-step", action="store_true", help="--serving reads every step's tokens before it launches the next")
    parser.add_argument("--peaks", action="store_true", help="measure this machine's read bandwidth and matrix-core rate with the library's probes")
    args = parser.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU: this engine has no multi-GPU path (asked for {args.gpus})")
        return 2

    if args.peaks:
        emit({"measured_peaks": measure_peaks(), "published": {"hbm_GBs": HBM_GBS, "mfma_bf16_TFLOPs": 2500.0, "mfma_fp32_TFLOPs": 157.3}}, args.json)
        return 0

    if args.serving:
        emit({"serving": measure_serving(args.dtype, args.temperature, not args.step_by_step)}, args.json)
        return 0

    from mini_llm_amd.config import config_from_dict
    from mini_llm_amd.engine.engine import Engine, EngineOptions
    from mini_llm_amd.engine.loading import build_model, require_gpu
    from mini_llm_amd.weights import bind_tensors, random_tensors

    shape, seed = SHAPES[args.shape]
    if args.context != CONTEXT:
        if args.context < 64:
            parser.error("--context must be at least 64")
        if args.prompt_len == PROMPT_LEN:
            args.prompt_len = args.context // 2
        globals()["CONTEXT"] = args.context
        shape = dict(shape, n_positions=args.context)
    if not 1 <= args.prompt_len < CONTEXT:
        parser.error(f"--prompt-len must be in 1..{CONTEXT - 1}")
    layers = args.layers or shape["n_layer"]
    config = config_from_dict(dict(shape, n_layer=layers))
    largest = max(args.batch, 1 if args.no_points else 64, 1 if args.no_check else 2)   # the check before timing runs two sequences
    tensors = {}

    def make_engine(dtype):
        """An engine over the seed's random weights (drawn once, on the host, and kept there for the check)."""
        model = build_model(config, dtype)
        if not tensors:
            tensors.update(random_tensors(model, seed))
        bind_tensors(model, tensors, require_gpu())
        return Engine(options=EngineOptions(dtype=dtype, max_sessions=largest, max_tokens=largest * CONTEXT, decode_lanes_from=args.lanes_from), model=model)

    def host_weights():
        return {name: tensor.numpy() for name, tensor in tensors.items()}

    engine = make_engine(args.dtype)
    checked = None if args.no_check else check_before_timing(engine, host_weights())
    if args.prefill_only:
        record = {"prefill": measure_prefill(engine, runs=max(args.steps, 1)), "dtype": args.dtype}
        if not args.no_kernels:
            record["kernels"] = measure_kernels(engine, decode=False)
        emit(record, args.json)
        return 0
    seconds, step_bytes = DecodeBench(engine, args.batch, args.prompt_len).run(args.steps, args.warmup)
    ms_per_step = seconds / args.steps * 1e3
    achieved = step_bytes / (seconds / args.steps) / 1e9
    short = {"bfloat16": "bf16", "float32": "fp32"}

    def check_record(values):
        if values is None:
            return None
        whole, plain = values
        return {"decode_vs_whole_prompt_scaled_diff": float(f"{whole:.3g}"), "decode_vs_plain_scaled_diff": None if plain is None else float(f"{plain:.3g}"),
                "tokens": 8}

    record = {
        "metric": f"decode tokens/s at batch {args.batch}, GPT-2 {args.shape}, {args.prompt_len}-token prompts decoding towards {CONTEXT}",
        "value": round(args.batch * args.steps / seconds, 1),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": short[args.dtype],
        "data": "synthetic: seeded random weights, uniform-random token ids",
        "config": {
            "model": f"gpt2-{args.shape}", "n_layer": shape["n_layer"], "layers_run": layers, "n_embd": config.n_embd,
            "n_head": config.n_head, "n_inner": config.n_inner, "vocab_size": config.vocab_size,
            "n_positions": config.n_positions, "activation_function": config.activation_function,
            "global_batch": args.batch, "prompt_len": args.prompt_len, "seq_len": CONTEXT, "page_size": engine.cache.page_size,
            "kv_cache_dtype": args.dtype, "sampling": "greedy", "parallelism": "single-gpu", "seed": seed,
        },
        "check": check_record(checked),
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_GBS, "unit": "GB/s", "frac": round(achieved / HBM_GBS, 4)},
    }
    if not args.no_points:
        record["prefill"] = measure_prefill(engine)
        points = {}
        for batch, steps in ((1, 128), (64, 64)):
            s, _ = DecodeBench(engine, batch, args.prompt_len).run(steps, 8)
            points[f"decode_b{batch}"] = round(batch * steps / s, 1)
        record["points"] = points
        record["kernels"] = measure_kernels(engine, batch=args.batch, context=(3 * CONTEXT // 4) // 64 * 64 + 8)
        if not args.one_dtype:
            # the same figures in the other precision (the headline names both): one record for the two
            other = "float32" if args.dtype == "bfloat16" else "bfloat16"
            del engine
            import torch

            torch.cuda.empty_cache()
            engine = make_engine(other)
            other_check = None if args.no_check else check_before_timing(engine, host_weights())
            figures = {}
            for batch, steps in ((1, 64), (args.batch, 64), (64, 32)):
                s, step_bytes = DecodeBench(engine, batch, args.prompt_len).run(steps, 8)
                figures[f"decode_b{batch}"] = round(batch * steps / s, 1)
                if batch == args.batch:
                    figures["ms_per_step"] = round(s / steps * 1e3, 4)
                    figures["roofline_frac"] = round(step_bytes / (s / steps) / 1e9 / HBM_GBS, 4)
            prefill = measure_prefill(engine)
            figures.update({"prefill": prefill["value"], "prefill_ms": prefill["ms"], "prefill_frac": prefill["frac"]})
            if other_check is not None:
                figures["check_vs_plain_scaled_diff"] = None if other_check[1] is None else float(f"{other_check[1]:.3g}")
            record[f"points_{short[other]}"] = figures
    emit(record, args.json)
    return 0


if __name__ == "__main__":
    sys.exit(main())

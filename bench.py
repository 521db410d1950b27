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


def measure_kernels(engine, batch: int = 8, context: int = 768, reps: int = 7):
    """What the kernels that a step's time goes to reach of their own roofline, each timed alone
    between two events over all layers' weights in turn (as a step walks them), median of ``reps``:
    for a 2,048-token prompt step the four products of a layer and the prompt attention (flops /
    time / the matrix cores' peak), for a decode step of ``batch`` sequences at ``context`` tokens the
    two halves of a layer and the head (the bytes each has to read / time / the memory's peak); a time
    holds the gap to the next kernel, as in a step. The
    reference prices its kernels the same way, against a pure read of the same bytes
    (docs/kernels/010_matvec_batch.md:20,108-117)."""
    import numpy as np
    import torch

    from mini_llm_amd.engine import StepEntry
    from mini_llm_amd.engine.batch import build_step_batch
    from mini_llm_amd.ops import kernels

    model, cache, runner = engine.model, engine.cache, engine.runner
    config, dtype = engine.config, engine.options.dtype
    e = element_size(dtype)
    compute = model.precision.compute
    d, ff, n_layer, vocab = config.n_embd, config.n_inner, config.n_layer, config.vocab_size
    rng = np.random.default_rng(SEED + 4)
    calls = [(model.blocks[call.block], cache.layer_context, call) for call in model.schedule]

    def timed(per_layer) -> float:
        """Seconds of one call of per_layer(block, ctx), averaged over the layers. The calls over the layers are captured into
        a graph and the replay is timed, as a step runs them: launched one by one the host's path through Python would count."""
        def over_the_layers():
            for block, context_of, call in calls:
                per_layer(block, context_of(batch_of_step, call))

        over_the_layers()
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            over_the_layers()
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        samples = []
        for rep in range(reps + 2):
            start.record()
            graph.replay()
            stop.record()
            torch.cuda.synchronize()
            samples.append(start.elapsed_time(stop) / 1e3 / len(calls))
        return float(np.median(samples[2:]))

    def staged(entries):
        """The batch of a step whose pages are reserved but which is never committed."""
        for entry in entries:
            cache.reserve(entry.request_id, len(entry.tokens))
        return build_step_batch(entries, cache, runner.staging, vocab_size=vocab, short_portion=model.short_portion())

    out = {}

    def note(name, seconds, work, peak, unit):
        out[name] = {"us": round(seconds * 1e6, 2), "frac": round(work / seconds / peak, 4), "of": unit}

    # --- a prompt step of two 1,024-token prompts
    lengths = [CONTEXT, CONTEXT]
    handles = [engine.try_take_cache() for _ in lengths]
    entries = [StepEntry(h, rng.integers(0, vocab, n).tolist(), [n - 1]) for h, n in zip(handles, lengths)]
    batch_of_step = staged(entries)
    rows = sum(lengths)
    hidden = model.embedding.forward(batch_of_step.tokens, batch_of_step.positions, model.position_encoding)
    block0 = model.blocks[0]
    mixer, feed = block0.mixer_part(), block0.feed_forward
    x = block0.norm_1.forward(hidden, compute)
    peak, unit = PEAK_FLOPS[dtype], f"{'bf16' if dtype == 'bfloat16' else 'fp32'} matrix peak"
    kept = {}

    def qkv(block, ctx):
        m = block.mixer_part()
        kept["q"] = kernels.linear_qkv_cache(x, m.qkv.weight, m.qkv.bias, ctx.k_pages, ctx.v_pages, ctx.group.slots, m.n_heads, m.n_kv_heads, m.head_size)

    note("prefill_qkv_product", timed(qkv), 2.0 * rows * d * 3 * d, peak, unit)

    def attention(block, ctx):
        m, b = block.mixer_part(), ctx.batch
        kept["mixed"] = kernels.paged_attention(kept["q"], ctx.k_pages, ctx.v_pages, b.token_request, b.positions, ctx.group.block_tables, m.n_heads,
                                                m.n_kv_heads, m.head_size, m.scale, max_q_len=b.max_q_len, max_len=b.max_total_len,
                                                q_starts=b.q_starts, context_lens=b.context_lens)

    note("prefill_attention", timed(attention), sum(4.0 * (n * (n + 1) / 2) * d for n in lengths), peak, unit)
    note("prefill_out_product", timed(lambda block, ctx: block.mixer_part().out.forward_pending(kept["mixed"], hidden)), 2.0 * rows * d * d, peak, unit)

    def up(block, ctx):
        kept["u"] = block.feed_forward.up.forward(x, activation=block.feed_forward.activation)

    note("prefill_up_product", timed(up), 2.0 * rows * d * ff, peak, unit)
    note("prefill_down_product", timed(lambda block, ctx: block.feed_forward.down.forward_pending(kept["u"], hidden)), 2.0 * rows * d * ff, peak, unit)
    kept.clear()
    for h in handles:
        cache.rollback(h)
        engine.release_cache(h)

    # --- a decode step: ``batch`` sequences that hold ``context`` tokens each
    handles = [engine.try_take_cache() for _ in range(batch)]
    for i in range(0, batch, 4):
        runner.step([StepEntry(h, rng.integers(0, vocab, context - 1).tolist(), []) for h in handles[i : i + 4]])
    entries = [StepEntry(h, [int(rng.integers(0, vocab))], [0]) for h in handles]
    batch_of_step = staged(entries)
    hidden = model.embedding.forward(batch_of_step.tokens, batch_of_step.positions, model.position_encoding)
    hbm = HBM_GBS * 1e9
    # each half takes the stream as the other half leaves it (with its last sums pending, where the parts do that)
    context_0 = cache.layer_context(batch_of_step, model.schedule[0])
    after_mlp = feed.forward_normed(hidden, block0.norm_2, compute, context_0)
    after_attention = mixer.forward_normed(after_mlp, block0.norm_1, compute, context_0)
    note("decode_attention_half", timed(lambda block, ctx: block.mixer_part().forward_normed(after_mlp, block.norm_1, compute, ctx)),
         (4.0 * d * d + batch * context * 2.0 * d) * e, hbm, "HBM peak")
    note("decode_mlp_half", timed(lambda block, ctx: block.feed_forward.forward_normed(after_attention, block.norm_2, compute, ctx)),
         2.0 * d * ff * e, hbm, "HBM peak")
    normed = model.final_norm.forward(kernels.settle(hidden), compute, row_index=batch_of_step.logit_rows)
    logits = {}

    def head(block, ctx):
        logits["rows"] = model.head.forward(normed)

    note("decode_head", timed(head), float(vocab) * d * e, hbm, "HBM peak")
    note("decode_sampler", timed(lambda block, ctx: kernels.sample(logits["rows"])), batch * vocab * 4.0, hbm, "HBM peak")
    for h in handles:
        cache.rollback(h)
        engine.release_cache(h)
    torch.cuda.synchronize()
    return out


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

    run_once()  # warm-up: captures the decode graphs
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
    parser.add_argument("--json", default=None, metavar="PATH", help="also write the printed record to this file (the reference's option)")
    parser.add_argument("--layers", type=int, default=None, help="run fewer layers than the configuration has (both numbers are reported)")
    parser.add_argument("--no-check", action="store_true", help="skip the comparison of decoding with a whole-prompt step before timing")
    parser.add_argument("--no-points", action="store_true", help="skip the batch 1 / batch 64 points, the prefill, the kernels and the other precision")
    parser.add_argument("--one-dtype", action="store_true", help="skip the figures in the other precision")
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
        emit({"prefill": measure_prefill(engine, runs=max(args.steps, 1)), "dtype": args.dtype}, args.json)
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
        "metric": f"decode tokens/s at batch {args.batch}, GPT-2 {args.shape}, {args.prompt_len}-token prompts decoding towards 1024",
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
        record["kernels"] = measure_kernels(engine)
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

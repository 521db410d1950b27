"""Each part alone against the plain implementation, at sizes of its own; and that parts and a
whole architecture defined in a test (a toy mixer with state of its own, another arrangement of
layers) can be registered, built and stepped without a change to the framework's files."""

import json
from dataclasses import dataclass

import numpy as np
import pytest
import torch

import plain_gpt2 as P
from conftest import random_tokens

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def bind_random(part, seed, dtype="float32"):
    """Draws the part's tensors by its own specs and binds them; returns them as float64 numpy
    in the stored layout (rounded as the part keeps them)."""
    from mini_llm_amd.precision import Precision
    from mini_llm_amd.weights.loader import place

    precision = Precision.from_name(dtype)
    rng = np.random.default_rng(seed)
    stored, placed = {}, {}
    for name, spec in part.named_tensor_specs().items():
        value = (spec.init.mean + 5 * spec.init.std * rng.standard_normal(spec.shape)).astype(np.float32)
        placed[name] = place(torch.from_numpy(value), spec, precision, DEV)
        if isinstance(placed[name], torch.Tensor):
            kept = placed[name].float().cpu().numpy()
            stored[name] = (kept.T if spec.keep_transposed else kept).astype(np.float64)
        else:  # a matrix in the packed layout of the kernels: the stored values, rounded as it keeps them
            stored[name] = torch.from_numpy(value).to(placed[name].dtype).float().numpy().astype(np.float64)
    part.bind_named(placed)
    return stored


def dev(a, dtype=torch.float32):
    return torch.as_tensor(np.asarray(a)).to(DEV).to(dtype).contiguous()


def host(t):
    return t.float().cpu().numpy().astype(np.float64)


def test_layernorm_part():
    from mini_llm_amd.parts import make_part

    part = make_part("norm", "layernorm", width=200, eps=3e-4)
    w = bind_random(part, 0)
    x = np.random.default_rng(1).standard_normal((6, 200)).astype(np.float32) * 0.01
    ref = P.layernorm(x.astype(np.float64), w["weight"], w["bias"], 3e-4)
    np.testing.assert_allclose(host(part.forward(dev(x), torch.float32)), ref, atol=2e-5, rtol=1e-5)
    assert np.abs(ref - P.layernorm(x.astype(np.float64), w["weight"], w["bias"], 1e-5)).max() > 1e-2  # eps is the part's


@pytest.mark.parametrize("stored_in_out", [True, False])
def test_linear_part_layouts(stored_in_out):
    from mini_llm_amd.parts import Linear

    part = Linear(72, 40, stored_in_out=stored_in_out)
    w = bind_random(part, 2)
    assert w["weight"].shape == ((72, 40) if stored_in_out else (40, 72)) and part.weight.shape == (40, 72)
    x = np.random.default_rng(3).standard_normal((9, 72)).astype(np.float32)
    matrix = w["weight"] if stored_in_out else w["weight"].T
    np.testing.assert_allclose(host(part.forward(dev(x))), x.astype(np.float64) @ matrix + w["bias"], atol=2e-5, rtol=1e-5)


@pytest.mark.parametrize("activation", ["gelu_new", "gelu"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_dense_mlp_part(activation, dtype):
    from mini_llm_amd.parts import make_part

    part = make_part("feed_forward", "dense_mlp", width=80, inner=200, activation=activation)
    w = bind_random(part, 4, dtype)
    rng = np.random.default_rng(5)
    x, r = rng.standard_normal((11, 80)).astype(np.float32), rng.standard_normal((11, 80)).astype(np.float32)
    td = torch.float32 if dtype == "float32" else torch.bfloat16
    xk = host(dev(x, td))
    ref = r + P.linear(P.ACTIVATIONS[activation](P.linear(xk, w["c_fc.weight"], w["c_fc.bias"])), w["c_proj.weight"], w["c_proj.bias"])
    out = part.forward(dev(x, td), dev(r))
    assert out.dtype == torch.float32
    tol = 2e-5 if dtype == "float32" else 3e-2
    np.testing.assert_allclose(host(out), ref, atol=tol, rtol=tol)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("rows", [20, 64, 65, 300])
def test_dense_mlp_with_a_long_inner_side(dtype, rows):
    # few output columns, a long inner side: the down product comes back cut along K, its sums
    # pending, and the next norm takes them
    from mini_llm_amd.ops import kernels
    from mini_llm_amd.parts import make_part

    width, inner, eps = 48, 1024, 1e-5
    part = make_part("feed_forward", "dense_mlp", width=width, inner=inner, activation="gelu_new")
    norm = make_part("norm", "layernorm", width=width, eps=eps)
    w, wn = bind_random(part, 14, dtype), bind_random(norm, 15)
    rng = np.random.default_rng(16)
    td = torch.float32 if dtype == "float32" else torch.bfloat16
    hidden = rng.standard_normal((rows, width)).astype(np.float32)

    class Portion:  # all the feed-forward asks of the batch: these rows are no single decoded tokens
        max_q_len = rows

    class Ctx:
        batch = Portion()

    out = part.forward_normed(dev(hidden), norm, td, Ctx())
    assert isinstance(out, kernels.PendingRows) and out.partials.shape[0] > 1
    x = host(dev(P.layernorm(hidden.astype(np.float64), wn["weight"], wn["bias"], eps), td))
    ref = hidden + P.linear(P.gelu_new(P.linear(x, w["c_fc.weight"], w["c_fc.bias"])), w["c_proj.weight"], w["c_proj.bias"])
    tol = 3e-5 if dtype == "float32" else 3e-2
    np.testing.assert_allclose(host(kernels.settle(out)), ref, atol=tol, rtol=tol)
    # and the norm that reads them next gives the sums back beside its own rows
    normed, summed = norm.forward_with_sums(out, torch.float32)
    np.testing.assert_allclose(host(summed), ref, atol=tol, rtol=tol)
    np.testing.assert_allclose(host(normed), P.layernorm(host(summed).astype(np.float64), wn["weight"], wn["bias"], eps), atol=1e-4, rtol=1e-4)


def test_embedding_positions_and_tied_head():
    from mini_llm_amd.parts import TiedHead, TokenEmbedding, make_part

    emb = TokenEmbedding(300, 48)
    pos = make_part("position_encoding", "learned", n_positions=20, width=48)
    we, wp = bind_random(emb, 6), bind_random(pos, 7)
    tokens, positions = [5, 299, 0, 17], [0, 19, 7, 7]
    out = emb.forward(dev(tokens, torch.int32), dev(positions, torch.int32), pos)
    np.testing.assert_allclose(host(out), we["weight"][tokens] + wp["weight"][positions], atol=1e-6)
    x = np.random.default_rng(8).standard_normal((3, 48)).astype(np.float32)
    np.testing.assert_allclose(host(TiedHead(emb).forward(dev(x))), P.lm_head(x.astype(np.float64), we["weight"]), atol=2e-5, rtol=1e-5)
    assert pos.max_positions() == 20


def make_cache_and_batch(mixers, portions, page_size=16, num_pages=24):
    """A cache for mixers (cache layer i for mixer i) and a batch of (request, context, new)."""
    from mini_llm_amd.cache import CacheManager
    from mini_llm_amd.engine.batch import BatchStaging, StepEntry, build_step_batch
    from mini_llm_amd.models.base import CacheGroupSpec

    groups = {}
    for i, m in enumerate(mixers):
        need = m.kv_need()
        groups.setdefault((need.n_kv_heads, need.head_size, need.window), []).append(i)
    specs = [CacheGroupSpec(f"g{j}", tuple(layers), *key) for j, (key, layers) in enumerate(groups.items())]
    cache = CacheManager(specs, {}, num_pages=num_pages, page_size=page_size, max_requests=8, dtype=torch.float32, device=DEV)
    return cache, BatchStaging(DEV)


def run_mixer_in_portions(mixer, cache, staging, sequences, cuts, layer=0):
    """Feeds each sequence's rows through the mixer in the given cuts; returns outputs per sequence."""
    from mini_llm_amd.engine.batch import StepEntry, build_step_batch
    from mini_llm_amd.models.base import LayerCall

    outs = {name: [] for name in sequences}
    fed = {name: 0 for name in sequences}
    for name in sequences:
        cache.open(name)
    for step in cuts:
        entries = [StepEntry(name, [0] * n, []) for name, n in step]
        for e in entries:
            cache.reserve(e.request_id, len(e.tokens))
        batch = build_step_batch(entries, cache, staging, vocab_size=1)
        sizes = dict(step)
        step = [(name, sizes[name]) for name in batch.request_ids]  # the rows lie in the batch's order: short portions first
        x = np.concatenate([sequences[name][fed[name] : fed[name] + n] for name, n in step])
        ctx = cache.layer_context(batch, LayerCall(0, layer))
        out = host(mixer.forward(dev(x), torch.zeros((len(x), x.shape[1]), device=DEV), ctx))
        at = 0
        for name, n in step:
            outs[name].append(out[at : at + n])
            at += n
            fed[name] += n
            cache.commit(name, n)
    return {name: np.concatenate(parts) for name, parts in outs.items()}


@pytest.mark.parametrize("n_heads,n_kv_heads,head_size,window", [(5, 5, 16, None), (4, 2, 32, None), (3, 3, 48, 21)])
def test_attention_part_in_portions(n_heads, n_kv_heads, head_size, window):
    from mini_llm_amd.parts import make_part

    width = 72
    mixer = make_part("mixer", "causal_attention", width=width, n_heads=n_heads, n_kv_heads=n_kv_heads, head_size=head_size, window=window)
    w = bind_random(mixer, 9)
    cache, staging = make_cache_and_batch([mixer], None)
    rng = np.random.default_rng(10)
    sequences = {"a": rng.standard_normal((50, width)).astype(np.float32), "b": rng.standard_normal((23, width)).astype(np.float32)}
    cuts = [[("a", 20)], [("a", 1), ("b", 17)], [("a", 13), ("b", 1)], [("b", 5), ("a", 16)]]
    got = run_mixer_in_portions(mixer, cache, staging, sequences, cuts)
    qw, kvw = n_heads * head_size, n_kv_heads * head_size
    for name, x in sequences.items():
        qkv = P.linear(x.astype(np.float64), w["c_attn.weight"], w["c_attn.bias"])
        a = P.multi_head_attention(qkv[:, :qw], qkv[:, qw : qw + kvw], qkv[:, qw + kvw :], n_heads, n_kv_heads, window)
        ref = P.linear(a, w["c_proj.weight"], w["c_proj.bias"])
        np.testing.assert_allclose(got[name], ref, atol=3e-5, rtol=1e-4, err_msg=name)


def test_pre_norm_block_part():
    from mini_llm_amd.parts import make_part

    width, heads, inner, eps = 64, 2, 100, 1e-3
    block = make_part(
        "block", "pre_norm",
        norm_1=make_part("norm", "layernorm", width=width, eps=eps),
        mixer=make_part("mixer", "causal_attention", width=width, n_heads=heads),
        norm_2=make_part("norm", "layernorm", width=width, eps=eps),
        feed_forward=make_part("feed_forward", "dense_mlp", width=width, inner=inner, activation="gelu"),
        compute_dtype=torch.float32,
    )
    w = bind_random(block, 11)
    cache, staging = make_cache_and_batch([block.mixer], None)
    x = np.random.default_rng(12).standard_normal((37, width)).astype(np.float32)

    class AsMixer:  # run_mixer_in_portions calls forward(x, residual, ctx)
        def forward(self, x, residual, ctx):
            return block.forward(x, ctx)

    got = run_mixer_in_portions(AsMixer(), cache, staging, {"s": x}, [[("s", 30)], [("s", 2)], [("s", 5)]])
    ref = P.block(x.astype(np.float64), w, heads, eps, "gelu")
    np.testing.assert_allclose(got["s"], ref, atol=5e-5, rtol=1e-4)


# ------------------------------------------------------------------------------------------------
# a toy architecture, defined here: a mixer with state of its own, different mixers in different
# layers, a layer that runs twice, and a layer that reads another layer's cache
# ------------------------------------------------------------------------------------------------
def define_toy():
    from mini_llm_amd.config import ModelConfig, register_architecture
    from mini_llm_amd.models import LayerCall, Model
    from mini_llm_amd.ops import kernels
    from mini_llm_amd.parts import Mixer, StateNeed, TiedHead, TokenEmbedding, make_part, register_part
    from mini_llm_amd.weights import VECTOR, Normal, TensorSpec

    class RunningMean(Mixer):
        """out[t] = gain * mean(x[0..t]) of the request; the state is (sum, count)."""

        def __init__(self, width):
            self.width = width
            self.gain = None

        def tensor_specs(self):
            return {"gain": TensorSpec((self.width,), VECTOR, Normal(0.3, mean=1.0))}

        def state_need(self):
            return StateNeed((self.width + 1,), torch.float32)

        def forward(self, x, residual, ctx):
            starts, slots = ctx.batch.host["q_starts"], ctx.batch.host["state_slots"]
            out = torch.empty((x.shape[0], self.width), dtype=torch.float32, device=x.device)
            for i, slot in enumerate(slots):
                rows = x[starts[i] : starts[i + 1]].float()
                state = ctx.state[slot]
                sums = state[: self.width] + torch.cumsum(rows, dim=0)
                counts = state[self.width] + torch.arange(1, rows.shape[0] + 1, device=x.device)
                out[starts[i] : starts[i + 1]] = sums / counts[:, None] * self.gain
                state[: self.width] = sums[-1]
                state[self.width] = counts[-1]
            return kernels.add(residual, out)

    register_part("mixer", "running_mean", RunningMean)

    @dataclass(frozen=True)
    class ToyConfig(ModelConfig):
        width: int
        heads: int
        inner: int
        vocab: int
        positions: int
        eps: float

        @classmethod
        def from_dict(cls, raw):
            return cls(raw["architectures"][0], raw["width"], raw["heads"], raw["inner"], raw["vocab"], raw["positions"], raw["eps"])

        def to_dict(self):
            return {"architectures": [self.architecture], "width": self.width, "heads": self.heads, "inner": self.inner,
                    "vocab": self.vocab, "positions": self.positions, "eps": self.eps}

    def build(config, precision):
        def block(mixer):
            return make_part(
                "block", "pre_norm",
                norm_1=make_part("norm", "layernorm", width=config.width, eps=config.eps), mixer=mixer,
                norm_2=make_part("norm", "layernorm", width=config.width, eps=config.eps),
                feed_forward=make_part("feed_forward", "dense_mlp", width=config.width, inner=config.inner, activation="gelu_new"),
                compute_dtype=precision.compute, names=("ln_1.", "mix.", "ln_2.", "mlp."))
        attention = lambda: make_part("mixer", "causal_attention", width=config.width, n_heads=config.heads)
        blocks = [block(make_part("mixer", "running_mean", width=config.width)), block(attention()), block(attention())]
        embedding = TokenEmbedding(config.vocab, config.width)
        return Model(
            config, precision, embedding=embedding,
            position_encoding=make_part("position_encoding", "learned", n_positions=config.positions, width=config.width),
            blocks=blocks,
            # layer 1 runs twice (a cache of its own each time); layer 2 reads what layer 1's first run stored
            schedule=[LayerCall(0, 0), LayerCall(1, 1), LayerCall(1, 2), LayerCall(2, 1, write_cache=False)],
            final_norm=make_part("norm", "layernorm", width=config.width, eps=config.eps), head=TiedHead(embedding),
            names={"embedding": "wte.", "position_encoding": "wpe.", "block": "layers.{i}.", "final_norm": "norm."},
        )

    register_architecture("ToyStateLM", ToyConfig, build)
    return ToyConfig


def plain_toy(raw, w, tokens):
    """The toy's forward pass from the plain implementation's functions."""
    d, eps, H = raw["width"], raw["eps"], raw["heads"]
    w = {k: v.astype(np.float64) for k, v in w.items()}
    L = lambda i, n: w[f"layers.{i}.{n}"]
    h = P.embed(tokens, w["wte.weight"], w["wpe.weight"])

    def mlp(i, r):
        ln2 = P.layernorm(r, L(i, "ln_2.weight"), L(i, "ln_2.bias"), eps)
        return r + P.linear(P.gelu_new(P.linear(ln2, L(i, "mlp.c_fc.weight"), L(i, "mlp.c_fc.bias"))), L(i, "mlp.c_proj.weight"), L(i, "mlp.c_proj.bias"))

    def attention(i, h, kv=None):
        qkv = P.linear(P.layernorm(h, L(i, "ln_1.weight"), L(i, "ln_1.bias"), eps), L(i, "mix.c_attn.weight"), L(i, "mix.c_attn.bias"))
        k, v = (qkv[:, d : 2 * d], qkv[:, 2 * d :]) if kv is None else kv
        a = P.multi_head_attention(qkv[:, :d], k, v, H)
        return h + P.linear(a, L(i, "mix.c_proj.weight"), L(i, "mix.c_proj.bias")), (k, v)

    ln1 = P.layernorm(h, L(0, "ln_1.weight"), L(0, "ln_1.bias"), eps)
    h = mlp(0, h + np.cumsum(ln1, axis=0) / np.arange(1, len(tokens) + 1)[:, None] * L(0, "mix.gain"))
    h, stored = attention(1, h)
    h = mlp(1, h)
    h, _ = attention(1, h)
    h = mlp(1, h)
    h, _ = attention(2, h, kv=stored)
    h = mlp(2, h)
    return P.lm_head(P.layernorm(h, w["norm.weight"], w["norm.bias"], eps), w["wte.weight"])


def test_toy_architecture_is_registered_built_and_stepped(tmp_path):
    from mini_llm_amd.config import load_config
    from mini_llm_amd.engine import ModelRunner, StepEntry
    from mini_llm_amd.engine.loading import load_model, make_cache
    from mini_llm_amd.weights import write_model_dir

    define_toy()
    raw = {"architectures": ["ToyStateLM"], "width": 48, "heads": 3, "inner": 72, "vocab": 211, "positions": 90, "eps": 1e-4}
    (tmp_path / "config.json").write_text(json.dumps(raw))
    config = load_config(tmp_path)                      # the registry finds the toy's configuration class
    write_model_dir(config, 3, tmp_path)                # random-weights mode over the toy's own tensors
    weights = P.read_safetensors(tmp_path / "model.safetensors")
    assert "layers.0.mix.gain" in weights and "layers.1.mix.c_attn.weight" in weights
    model = load_model(tmp_path, "float32")
    assert model.state_needs().keys() == {0} and [g.layers for g in model.cache_groups()] == [(1, 2)]
    cache = make_cache(model, max_tokens=256, page_size=16, max_requests=4)
    runner = ModelRunner(model, cache, DEV)
    seqs = {"a": random_tokens(1, 70, 211), "b": random_tokens(2, 33, 211)}
    ref = {name: plain_toy(raw, weights, t) for name, t in seqs.items()}
    got = {name: [] for name in seqs}
    for name in seqs:
        cache.open(name)
    cuts = [[("a", 30)], [("a", 1), ("b", 20)], [("b", 2), ("a", 2)], [("a", 37), ("b", 11)]]
    fed = {name: 0 for name in seqs}
    for step in cuts:
        entries = [StepEntry(name, seqs[name][fed[name] : fed[name] + n], list(range(n))) for name, n in step]
        logits = host(runner.step(entries))
        at = 0
        for name, n in step:
            got[name].append(logits[at : at + n])
            at += n
            fed[name] += n
    for name in seqs:
        np.testing.assert_allclose(np.concatenate(got[name]), ref[name], atol=5e-5, rtol=2e-4, err_msg=name)
    # a new request in a used slot starts from a cleared state
    cache.close("a")
    cache.open("c")
    again = host(runner.step([StepEntry("c", seqs["a"], [69])]))
    np.testing.assert_allclose(again[0], ref["a"][69], atol=5e-5, rtol=2e-4)


# ------------------------------------------------------------------------------------------------
# a second toy, defined here: positions that enter inside a mixer (no table at the embedding) and
# a feed-forward that routes each row to one of two experts built from the framework's own parts
# ------------------------------------------------------------------------------------------------
def define_routed_toy():
    from mini_llm_amd.config import ModelConfig, register_architecture
    from mini_llm_amd.models import LayerCall, Model
    from mini_llm_amd.ops import kernels
    from mini_llm_amd.parts import FeedForward, Mixer, PositionEncoding, TiedHead, TokenEmbedding, make_part, register_part
    from mini_llm_amd.weights import VECTOR, Normal, TensorSpec

    class PhaseEncoding(PositionEncoding):
        """x[t] * cos(position t * rate), applied by the mixer that holds it."""

        stage = "mixer"

        def __init__(self, n_positions, width):
            self.n_positions, self.width = n_positions, width
            self.rate = None

        def tensor_specs(self):
            return {"rate": TensorSpec((self.width,), VECTOR, Normal(0.05))}

        def max_positions(self):
            return self.n_positions

        def apply(self, x, positions):
            return x * torch.cos(positions[:, None].float() * self.rate)

    class PhasedGate(Mixer):
        def __init__(self, width, encoding):
            self.width, self.encoding = width, encoding   # the encoding's tensor belongs to the model, not to this part
            self.gain = None

        def tensor_specs(self):
            return {"gain": TensorSpec((self.width,), VECTOR, Normal(0.3, mean=1.0))}

        def forward(self, x, residual, ctx):
            positions = ctx.batch.positions[: x.shape[0]]
            return kernels.add(residual, (self.encoding.apply(x.float(), positions) * self.gain).contiguous())

    class TwoExperts(FeedForward):
        graph_safe = False  # it plans on the host

        def __init__(self, width, inner):
            self.width = width
            self.experts = [make_part("feed_forward", "dense_mlp", width=width, inner=inner, activation="gelu_new") for _ in range(2)]
            self.router = None

        def tensor_specs(self):
            return {"router": TensorSpec((self.width,), VECTOR, Normal(1.0))}

        def children(self):
            return {f"experts.{e}.": expert for e, expert in enumerate(self.experts)}

        def forward(self, x, residual):
            chosen = (x.float() @ self.router) > 0   # router logits in 32-bit
            out = torch.empty_like(residual)
            for e, expert in enumerate(self.experts):
                rows = torch.nonzero(chosen == bool(e)).flatten()
                if rows.numel():
                    out[rows] = kernels.settle(expert.forward(x[rows].contiguous(), residual[rows].contiguous()))
            return out

    register_part("position_encoding", "phase", PhaseEncoding)
    register_part("mixer", "phased_gate", PhasedGate)
    register_part("feed_forward", "two_experts", TwoExperts)

    @dataclass(frozen=True)
    class RoutedConfig(ModelConfig):
        width: int
        heads: int
        inner: int
        vocab: int
        positions: int
        eps: float

        @classmethod
        def from_dict(cls, raw):
            return cls(raw["architectures"][0], raw["width"], raw["heads"], raw["inner"], raw["vocab"], raw["positions"], raw["eps"])

        def to_dict(self):
            return {"architectures": [self.architecture], "width": self.width, "heads": self.heads, "inner": self.inner,
                    "vocab": self.vocab, "positions": self.positions, "eps": self.eps}

    def build(config, precision):
        norm = lambda: make_part("norm", "layernorm", width=config.width, eps=config.eps)
        encoding = make_part("position_encoding", "phase", n_positions=config.positions, width=config.width)
        names = ("ln_1.", "mix.", "ln_2.", "mlp.")
        blocks = [
            make_part("block", "pre_norm", norm_1=norm(), mixer=make_part("mixer", "phased_gate", width=config.width, encoding=encoding),
                      norm_2=norm(), feed_forward=make_part("feed_forward", "two_experts", width=config.width, inner=config.inner),
                      compute_dtype=precision.compute, names=names),
            make_part("block", "pre_norm", norm_1=norm(), mixer=make_part("mixer", "causal_attention", width=config.width, n_heads=config.heads),
                      norm_2=norm(), feed_forward=make_part("feed_forward", "dense_mlp", width=config.width, inner=config.inner, activation="gelu"),
                      compute_dtype=precision.compute, names=names),
        ]
        embedding = TokenEmbedding(config.vocab, config.width)
        return Model(config, precision, embedding=embedding, position_encoding=encoding, blocks=blocks,
                     schedule=[LayerCall(0, 0), LayerCall(1, 1)], final_norm=norm(), head=TiedHead(embedding),
                     names={"embedding": "wte.", "position_encoding": "phase.", "block": "layers.{i}.", "final_norm": "norm."})

    register_architecture("ToyRoutedLM", RoutedConfig, build)


def plain_routed_toy(raw, w, tokens):
    d, eps, H = raw["width"], raw["eps"], raw["heads"]
    w = {k: v.astype(np.float64) for k, v in w.items()}
    L = lambda i, n: w[f"layers.{i}.{n}"]
    mlp = lambda x, prefix, act: P.linear(act(P.linear(x, w[prefix + "c_fc.weight"], w[prefix + "c_fc.bias"])), w[prefix + "c_proj.weight"], w[prefix + "c_proj.bias"])
    h = w["wte.weight"][tokens]                                              # no position table
    positions = np.arange(len(tokens))[:, None]
    h = h + P.layernorm(h, L(0, "ln_1.weight"), L(0, "ln_1.bias"), eps) * np.cos(positions * w["phase.rate"]) * L(0, "mix.gain")
    ln2 = P.layernorm(h, L(0, "ln_2.weight"), L(0, "ln_2.bias"), eps)
    scores = ln2 @ L(0, "mlp.router")
    assert np.abs(scores).min() > 1e-3, "a router score too close to the border for a comparison"
    experts = [mlp(ln2, f"layers.0.mlp.experts.{e}.", P.gelu_new) for e in range(2)]
    h = h + np.where((scores > 0)[:, None], experts[1], experts[0])
    qkv = P.linear(P.layernorm(h, L(1, "ln_1.weight"), L(1, "ln_1.bias"), eps), L(1, "mix.c_attn.weight"), L(1, "mix.c_attn.bias"))
    h = h + P.linear(P.multi_head_attention(qkv[:, :d], qkv[:, d : 2 * d], qkv[:, 2 * d :], H), L(1, "mix.c_proj.weight"), L(1, "mix.c_proj.bias"))
    h = h + mlp(P.layernorm(h, L(1, "ln_2.weight"), L(1, "ln_2.bias"), eps), "layers.1.mlp.", P.ACTIVATIONS["gelu"])
    return P.lm_head(P.layernorm(h, w["norm.weight"], w["norm.bias"], eps), w["wte.weight"])


def test_toy_with_positions_inside_a_mixer_and_a_routed_feed_forward(tmp_path):
    from mini_llm_amd.config import load_config
    from mini_llm_amd.engine import ModelRunner, StepEntry
    from mini_llm_amd.engine.loading import load_model, make_cache
    from mini_llm_amd.weights import write_model_dir

    define_routed_toy()
    raw = {"architectures": ["ToyRoutedLM"], "width": 64, "heads": 2, "inner": 56, "vocab": 150, "positions": 80, "eps": 1e-5}
    (tmp_path / "config.json").write_text(json.dumps(raw))
    config = load_config(tmp_path)
    write_model_dir(config, 5, tmp_path)
    weights = P.read_safetensors(tmp_path / "model.safetensors")
    assert {"phase.rate", "layers.0.mix.gain", "layers.0.mlp.router", "layers.0.mlp.experts.1.c_proj.weight"} <= weights.keys()
    assert not any(name.startswith("wpe") for name in weights)
    model = load_model(tmp_path, "float32")
    assert model.max_positions() == 80 and [g.layers for g in model.cache_groups()] == [(1,)]
    cache = make_cache(model, max_tokens=256, page_size=16, max_requests=4)
    runner = ModelRunner(model, cache, DEV)
    assert not runner.use_graphs                          # the routed feed-forward plans on the host
    seqs = {"a": random_tokens(3, 60, 150), "b": random_tokens(4, 25, 150)}
    ref = {name: plain_routed_toy(raw, weights, t) for name, t in seqs.items()}
    got, fed = {name: [] for name in seqs}, {name: 0 for name in seqs}
    for name in seqs:
        cache.open(name)
    # portions of both kinds in one step, so that the rows are not laid out in the order given
    for step in [[("a", 20), ("b", 3)], [("b", 1), ("a", 9)], [("a", 1), ("b", 1)], [("b", 20), ("a", 30)]]:
        entries = [StepEntry(name, seqs[name][fed[name] : fed[name] + n], list(range(n))) for name, n in step]
        logits = host(runner.step(entries))
        at = 0
        for name, n in step:
            got[name].append(logits[at : at + n])
            at += n
            fed[name] += n
    for name in seqs:
        np.testing.assert_allclose(np.concatenate(got[name]), ref[name], atol=5e-5, rtol=2e-4, err_msg=name)


# ------------------------------------------------------------------------------------------------
# a third toy: no position encoding at all, so the model has no limit of its own and the engine's
# caller has to name the longest sequence
# ------------------------------------------------------------------------------------------------
def define_unbounded_toy():
    from mini_llm_amd.config import ModelConfig, register_architecture
    from mini_llm_amd.models import LayerCall, Model
    from mini_llm_amd.parts import TiedHead, TokenEmbedding, make_part

    @dataclass(frozen=True)
    class UnboundedConfig(ModelConfig):
        width: int
        heads: int
        inner: int
        vocab: int
        eps: float

        @classmethod
        def from_dict(cls, raw):
            return cls(raw["architectures"][0], raw["width"], raw["heads"], raw["inner"], raw["vocab"], raw["eps"])

        def to_dict(self):
            return {"architectures": [self.architecture], "width": self.width, "heads": self.heads, "inner": self.inner,
                    "vocab": self.vocab, "eps": self.eps}

    def build(config, precision):
        norm = lambda: make_part("norm", "layernorm", width=config.width, eps=config.eps)
        block = lambda: make_part(
            "block", "pre_norm", norm_1=norm(), mixer=make_part("mixer", "causal_attention", width=config.width, n_heads=config.heads),
            norm_2=norm(), feed_forward=make_part("feed_forward", "dense_mlp", width=config.width, inner=config.inner, activation="gelu_new"),
            compute_dtype=precision.compute, names=("ln_1.", "mix.", "ln_2.", "mlp."))
        embedding = TokenEmbedding(config.vocab, config.width)
        return Model(config, precision, embedding=embedding, position_encoding=None, blocks=[block(), block()],
                     schedule=[LayerCall(0, 0), LayerCall(1, 1)], final_norm=norm(), head=TiedHead(embedding),
                     names={"embedding": "wte.", "block": "layers.{i}.", "final_norm": "norm."})

    register_architecture("ToyUnboundedLM", UnboundedConfig, build)


def plain_unbounded_toy(raw, w, tokens):
    d, eps, H = raw["width"], raw["eps"], raw["heads"]
    w = {k: v.astype(np.float64) for k, v in w.items()}
    h = w["wte.weight"][tokens]
    for i in range(2):
        layer = {name[len(f"layers.{i}."):].replace("mix.", "attn."): t for name, t in w.items() if name.startswith(f"layers.{i}.")}
        h = P.block(h, layer, H, eps, "gelu_new")
    return P.lm_head(P.layernorm(h, w["norm.weight"], w["norm.bias"], eps), w["wte.weight"])


def test_engine_over_a_model_without_a_position_limit(tmp_path):
    from mini_llm_amd.config import load_config
    from mini_llm_amd.engine.engine import Engine, EngineOptions
    from mini_llm_amd.engine.loading import load_model
    from mini_llm_amd.weights import write_model_dir

    define_unbounded_toy()
    raw = {"architectures": ["ToyUnboundedLM"], "width": 64, "heads": 4, "inner": 80, "vocab": 190, "eps": 1e-5}
    (tmp_path / "config.json").write_text(json.dumps(raw))
    write_model_dir(load_config(tmp_path), 9, tmp_path)
    weights = P.read_safetensors(tmp_path / "model.safetensors")
    assert not any(name.startswith("wpe") for name in weights)
    model = load_model(tmp_path, "float32")
    assert model.max_positions() is None
    # nothing says how long a sequence may get: refused, also with the pool's size given
    for options in (EngineOptions(dtype="float32", max_sessions=3), EngineOptions(dtype="float32", max_sessions=3, max_tokens=512),
                    EngineOptions(dtype="float32", max_sessions=3, cache_gib=0.01)):
        with pytest.raises(ValueError, match="max_length"):
            Engine(model=model, options=options)
    engine = Engine(model=model, options=EngineOptions(dtype="float32", max_sessions=3, max_length=96, page_size=16, max_tokens_per_step=20))
    assert engine.cache.max_length == 96 and engine.cache.max_blocks() == 6
    assert engine.cache.free_pages() == [3 * 6]           # max_sessions sequences of max_length
    assert engine.runner.use_graphs                        # its decode steps are captured like any other model's
    prompts = [random_tokens(40 + i, n, 190) for i, n in enumerate((3, 31, 50, 17))]
    generated = engine.generate(prompts, max_new_tokens=12)
    assert engine.runner.graph_steps > 0
    for prompt, new in zip(prompts, generated):
        tokens = list(prompt)
        for token in new:
            logits = plain_unbounded_toy(raw, weights, tokens)[-1]
            assert logits[token] >= logits.max() - 1e-5, (len(tokens), token, int(logits.argmax()))
            tokens.append(token)
        assert len(new) == 12
    # the caller's limit ends a request as a model's own would
    from mini_llm_amd.engine.scheduler import Request

    got = []
    engine.submit(Request(random_tokens(50, 90, 190), on_token=lambda token, finish: got.append(finish), on_error=got.append, max_new_tokens=30))
    engine.scheduler.run_until_idle()
    assert got == [None] * 5 + ["context"]
    engine.close()

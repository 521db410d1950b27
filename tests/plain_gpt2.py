"""A plain, slow GPT-2 forward pass: whole sequences, no cache, one function per part.

Written from the formulas of WillyBruhn/mini_llm's CPU engine (every function cites the file and
lines it follows). It shares no code with ``mini_llm_amd``: tests compare the engine with it.
Everything is numpy; ``dtype`` is the precision of the arithmetic (float64 by default, so that the
oracle's own rounding is far below the engine's).
"""

from __future__ import annotations

import json
import math
import struct
from pathlib import Path

import numpy as np


# --------------------------------------------------------------------------------------------
# parts
# --------------------------------------------------------------------------------------------
def embed(tokens, wte, wpe, first_position=0):
    """h[t] = wte[token[t]] + wpe[first_position + t]  (engine/src/embedding.c:9-16; the offset
    is the cache length in the decode path, engine/src/gpt2_gpu.cu:321)."""
    tokens = np.asarray(tokens, dtype=np.int64)
    positions = first_position + np.arange(len(tokens))
    return wte[tokens] + wpe[positions]


def layernorm(x, gamma, beta, eps):
    """Row norm with a centred, biased variance (engine/src/layernorm.c:15-33):
    mean = sum(x)/n; var = sum((x-mean)^2)/n; y = (x-mean) * 1/sqrt(var+eps) * gamma + beta."""
    n = x.shape[-1]
    mean = x.sum(axis=-1, keepdims=True) / n
    diff = x - mean
    var = (diff * diff).sum(axis=-1, keepdims=True) / n
    inv = 1.0 / np.sqrt(var + eps)
    return diff * inv * gamma + beta


def linear(x, weight, bias):
    """y = x @ W + b with W in Conv1D layout [in, out], no transpose
    (engine/src/matrixmult.c:9-18, engine/src/linear.c:5-18)."""
    y = x @ weight
    if bias is not None:
        y = y + bias
    return y


def gelu_new(x):
    """tanh GELU: 0.5*x*(1+tanh(0.7978845608*(x+0.044715*x^3)))  (engine/src/gelu.c:11-20)."""
    return 0.5 * x * (1.0 + np.tanh(0.7978845608028654 * (x + 0.044715 * x * x * x)))


def gelu_erf(x):
    """exact GELU: 0.5*x*(1+erf(x/sqrt(2)))  (engine/src/gelu.c:5-9)."""
    erf = np.vectorize(math.erf, otypes=[np.float64])
    return (0.5 * x * (1.0 + erf(np.asarray(x, dtype=np.float64) / math.sqrt(2.0)))).astype(x.dtype)


ACTIVATIONS = {"gelu_new": gelu_new, "gelu": gelu_erf}


def causal_softmax(scores, window=None):
    """Row softmax over keys j <= i (engine/src/softmax.c:29-55): p = exp(s-max)/sum(exp(s-max)),
    the maximum and the sum taken over the allowed keys only. ``window`` (not in the reference,
    which has full attention only) further limits row i to keys j > i - window."""
    rows, cols = scores.shape
    out = np.zeros_like(scores)
    for i in range(rows):
        last = min(i, cols - 1)
        first = 0 if window is None else max(0, i - window + 1)
        row = scores[i, first : last + 1]
        e = np.exp(row - row.max())
        out[i, first : last + 1] = e / e.sum()
    return out


def attention_head(q, k, v, window=None):
    """One head, causal: s[i,j] = q_i.k_j / sqrt(head_size); softmax over j<=i; out = p @ v
    (engine/src/attention.c:8-54)."""
    head_size = q.shape[-1]
    scores = (q @ k.T) / math.sqrt(head_size)
    return causal_softmax(scores, window) @ v


def multi_head_attention(q, k, v, n_head, n_kv_head=None, window=None):
    """Head h owns columns [h*hs, (h+1)*hs) of q and of the output (engine/src/attention.c:56-104).
    The reference has as many key/value heads as query heads; with fewer (``n_kv_head``), query
    head h reads key/value head h // (n_head // n_kv_head)."""
    n_kv_head = n_head if n_kv_head is None else n_kv_head
    hs = q.shape[-1] // n_head
    out = np.zeros_like(q)
    for h in range(n_head):
        g = h // (n_head // n_kv_head)
        out[:, h * hs : (h + 1) * hs] = attention_head(
            q[:, h * hs : (h + 1) * hs], k[:, g * hs : (g + 1) * hs], v[:, g * hs : (g + 1) * hs], window
        )
    return out


def _keep(x):
    return x


def block(x, w, n_head, eps, activation, stored=_keep):
    """Pre-norm block in the reference's order (engine/src/transformer_block.c:49-71):
    ln_1 -> q,k,v (columns of the fused c_attn, engine/src/gpt2.c:79-90) -> attention -> c_proj ->
    residual add -> ln_2 -> c_fc -> activation -> mlp.c_proj -> residual add.

    ``stored`` is applied to every tensor a reduced-precision run keeps between kernels (norm
    outputs, q/k/v, the attention output, the activated MLP row); the residual stream is not one
    of them. The reference keeps everything in 32-bit, which is the default here."""
    d = x.shape[-1]
    ln1 = stored(layernorm(x, w["ln_1.weight"], w["ln_1.bias"], eps))
    qkv = stored(linear(ln1, w["attn.c_attn.weight"], w["attn.c_attn.bias"]))
    q, k, v = qkv[:, :d], qkv[:, d : 2 * d], qkv[:, 2 * d :]
    a = stored(multi_head_attention(q, k, v, n_head))
    r = x + linear(a, w["attn.c_proj.weight"], w["attn.c_proj.bias"])
    ln2 = stored(layernorm(r, w["ln_2.weight"], w["ln_2.bias"], eps))
    u = stored(ACTIVATIONS[activation](linear(ln2, w["mlp.c_fc.weight"], w["mlp.c_fc.bias"])))
    return r + linear(u, w["mlp.c_proj.weight"], w["mlp.c_proj.bias"])


def lm_head(x, wte):
    """logits[t, v] = x[t] . wte[v]: tied to the token table, no bias (engine/src/gpt2.c:244-256)."""
    return x @ wte.T


# --------------------------------------------------------------------------------------------
# whole model
# --------------------------------------------------------------------------------------------
def forward(config: dict, weights: dict, tokens, dtype=np.float64, stored=_keep, block_outputs=None):
    """Logits [len(tokens), vocab] of one whole sequence (engine/src/gpt2.c:198-262): embed,
    n_layer blocks, ln_f on every row, tied head. ``stored``: see ``block``. ``block_outputs``: a
    list that receives the embedding and then every block's output (as the reference can hand out
    its blocks' outputs: engine/src/gpt2.c:234-237)."""
    w = {name: np.asarray(t, dtype=dtype) for name, t in weights.items()}
    n_layer = config["n_layer"]
    eps = config.get("layer_norm_epsilon", 1e-5)
    activation = config.get("activation_function", "gelu_new")
    if len(tokens) > config["n_positions"]:
        raise ValueError("sequence longer than n_positions")
    h = embed(tokens, w["wte.weight"], w["wpe.weight"])
    if block_outputs is not None:
        block_outputs.append(h)
    for i in range(n_layer):
        prefix = f"h.{i}."
        layer = {k[len(prefix) :]: t for k, t in w.items() if k.startswith(prefix)}
        h = block(h, layer, config["n_head"], eps, activation, stored)
        if block_outputs is not None:
            block_outputs.append(h)
    h = stored(layernorm(h, w["ln_f.weight"], w["ln_f.bias"], eps))
    return lm_head(h, w["wte.weight"])


def greedy(config, weights, prompt, n_new, dtype=np.float64):
    """Greedy continuation by recomputing the whole sequence for every token (the reference's
    RecomputeSession, pytorch/src/mini_llm/native.py:41-55); argmax takes the first maximum
    (engine/include/argmax.h:10-13)."""
    tokens = list(prompt)
    for _ in range(n_new):
        tokens.append(int(np.argmax(forward(config, weights, tokens, dtype)[-1])))
    return tokens[len(prompt) :]


# --------------------------------------------------------------------------------------------
# sampling (the completion script samples with temperature and top-p, scripts/complete.py:116-123)
# --------------------------------------------------------------------------------------------
def softmax(x):
    """engine/src/softmax.c:5-27."""
    e = np.exp(x - x.max(axis=-1, keepdims=True))
    return e / e.sum(axis=-1, keepdims=True)


def top_p_keep(probs, top_p):
    """Nucleus: token i is kept if the probability mass of all strictly more likely tokens is
    below top_p (the smallest set of most likely tokens whose mass reaches top_p; equal
    probabilities stand or fall together)."""
    probs = np.asarray(probs, dtype=np.float64)
    keep = np.zeros(len(probs), dtype=bool)
    for i, p in enumerate(probs):
        keep[i] = probs[probs > p].sum() < top_p
    return keep


# --------------------------------------------------------------------------------------------
# own reader/writer of model folders, so that tests do not lean on the engine's loader
# --------------------------------------------------------------------------------------------
_ST_DTYPES = {"F32": np.float32, "F64": np.float64, "I32": np.int32, "I64": np.int64, "F16": np.float16}


def _bf16_bytes_to_f32(raw: bytes) -> np.ndarray:
    u16 = np.frombuffer(raw, dtype="<u2").astype(np.uint32)
    return (u16 << 16).view(np.float32)


def f32_to_bf16_rne(x: np.ndarray) -> np.ndarray:
    """float32 -> bfloat16 (as uint16), round to nearest even."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    rounded = (u + 0x7FFF + ((u >> 16) & 1)) >> 16
    return rounded.astype(np.uint16)


def round_to_bf16(x: np.ndarray) -> np.ndarray:
    """The float32 value nearest-even rounded to bfloat16 precision."""
    return (f32_to_bf16_rne(x).astype(np.uint32) << 16).view(np.float32).reshape(np.shape(x))


def stored_as_bf16(x: np.ndarray) -> np.ndarray:
    """``stored`` for a bfloat16 run: values rounded to bfloat16, arithmetic type kept."""
    return round_to_bf16(np.asarray(x, dtype=np.float32)).astype(x.dtype)


def bf16_weights(weights: dict) -> dict:
    """The tensors as a bfloat16 run keeps them: matrices and tables rounded, vectors untouched."""
    return {k: round_to_bf16(v) if v.ndim == 2 else v for k, v in weights.items()}


def read_safetensors(path) -> dict:
    raw = Path(path).read_bytes()
    (hlen,) = struct.unpack("<Q", raw[:8])
    header = json.loads(raw[8 : 8 + hlen])
    out = {}
    for name, info in header.items():
        if name == "__metadata__":
            continue
        a, b = info["data_offsets"]
        buf = raw[8 + hlen + a : 8 + hlen + b]
        if info["dtype"] == "BF16":
            arr = _bf16_bytes_to_f32(buf)
        else:
            arr = np.frombuffer(buf, dtype=_ST_DTYPES[info["dtype"]])
        out[name] = arr.reshape(info["shape"])
    return out


def write_safetensors(path, tensors: dict, bf16: bool = False) -> None:
    header, chunks, offset = {}, [], 0
    for name, arr in tensors.items():
        arr = np.ascontiguousarray(arr)
        if bf16 and arr.dtype == np.float32:
            data, dt = f32_to_bf16_rne(arr).tobytes(), "BF16"
        else:
            dt = {v: k for k, v in _ST_DTYPES.items()}[arr.dtype.type]
            data = arr.tobytes()
        header[name] = {"dtype": dt, "shape": list(arr.shape), "data_offsets": [offset, offset + len(data)]}
        chunks.append(data)
        offset += len(data)
    hjson = json.dumps(header, separators=(",", ":")).encode()
    hjson += b" " * (-len(hjson) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(hjson)))
        f.write(hjson)
        for c in chunks:
            f.write(c)


def strip_prefix(tensors: dict) -> dict:
    """Names without the ``transformer.`` prefix; masks and a tied ``lm_head.weight`` dropped."""
    out = {}
    for name, t in tensors.items():
        if name.startswith("transformer."):
            name = name[len("transformer.") :]
        if name == "lm_head.weight" or name.endswith(".attn.bias") or name.endswith(".attn.masked_bias"):
            continue
        out[name] = t
    return out


def load_model_dir(path):
    path = Path(path)
    config = json.loads((path / "config.json").read_text())
    if config.get("n_inner") is None:
        config["n_inner"] = 4 * config["n_embd"]
    return config, strip_prefix(read_safetensors(path / "model.safetensors"))


def random_weights(config: dict, seed: int) -> dict:
    """Random GPT-2 tensors (float32), by the recipe the benchmark configurations name: tables and
    matrices N(0, 0.02); the two c_proj matrices N(0, 0.02/sqrt(2*n_layer)); biases N(0, 0.01);
    norm gains 1 + N(0, 0.05), norm offsets N(0, 0.02). The generator is this file's own."""
    rng = np.random.default_rng(seed)
    d, L, V, P = config["n_embd"], config["n_layer"], config["vocab_size"], config["n_positions"]
    ff = config.get("n_inner") or 4 * d

    def n(shape, std, mean=0.0):
        return (mean + std * rng.standard_normal(shape)).astype(np.float32)

    w = {"wte.weight": n((V, d), 0.02), "wpe.weight": n((P, d), 0.02)}
    proj_std = 0.02 / math.sqrt(2 * L)
    for i in range(L):
        p = f"h.{i}."
        w[p + "ln_1.weight"] = n((d,), 0.05, 1.0)
        w[p + "ln_1.bias"] = n((d,), 0.02)
        w[p + "attn.c_attn.weight"] = n((d, 3 * d), 0.02)
        w[p + "attn.c_attn.bias"] = n((3 * d,), 0.01)
        w[p + "attn.c_proj.weight"] = n((d, d), proj_std)
        w[p + "attn.c_proj.bias"] = n((d,), 0.01)
        w[p + "ln_2.weight"] = n((d,), 0.05, 1.0)
        w[p + "ln_2.bias"] = n((d,), 0.02)
        w[p + "mlp.c_fc.weight"] = n((d, ff), 0.02)
        w[p + "mlp.c_fc.bias"] = n((ff,), 0.01)
        w[p + "mlp.c_proj.weight"] = n((ff, d), proj_std)
        w[p + "mlp.c_proj.bias"] = n((d,), 0.01)
    w["ln_f.weight"] = n((d,), 0.05, 1.0)
    w["ln_f.bias"] = n((d,), 0.02)
    return w


# --- the framework's documented random-weights generator, written out a second time -----------------
# (its definition: mini_llm_amd/weights/counter_rng.py's docstring; integers here are Python's own)
def counter_normal(seed: int, name: str, count: int) -> np.ndarray:
    """n(0) .. n(count - 1) of tensor ``name`` under ``seed``, float64."""
    m = (1 << 64) - 1

    def mix(z):
        z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & m
        z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & m
        return z ^ (z >> 31)

    h = 0xCBF29CE484222325
    for byte in name.encode("utf-8"):
        h = ((h ^ byte) * 0x100000001B3) & m
    key = mix(mix(seed & m) ^ h)
    g = 0x9E3779B97F4A7C15
    a = np.array([mix((key + (2 * i + 1) * g) & m) >> 12 for i in range(count)], dtype=np.float64)
    b = np.array([mix((key + (2 * i + 2) * g) & m) >> 12 for i in range(count)], dtype=np.float64)
    u1, u2 = (a + 0.5) / 2.0**52, (b + 0.5) / 2.0**52
    return np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * np.pi * u2)


def counter_random_weights(config: dict, seed: int) -> dict:
    """The tensors the framework's random-weights mode writes for this configuration and seed."""
    d, L, V, P = config["n_embd"], config["n_layer"], config["vocab_size"], config["n_positions"]
    ff = config.get("n_inner") or 4 * d
    proj_std = 0.02 / math.sqrt(2 * L)
    recipe = {"wte.weight": ((V, d), 0.0, 0.02), "wpe.weight": ((P, d), 0.0, 0.02),
              "ln_f.weight": ((d,), 1.0, 0.05), "ln_f.bias": ((d,), 0.0, 0.02)}
    for i in range(L):
        p = f"h.{i}."
        recipe.update({
            p + "ln_1.weight": ((d,), 1.0, 0.05), p + "ln_1.bias": ((d,), 0.0, 0.02),
            p + "attn.c_attn.weight": ((d, 3 * d), 0.0, 0.02), p + "attn.c_attn.bias": ((3 * d,), 0.0, 0.01),
            p + "attn.c_proj.weight": ((d, d), 0.0, proj_std), p + "attn.c_proj.bias": ((d,), 0.0, 0.01),
            p + "ln_2.weight": ((d,), 1.0, 0.05), p + "ln_2.bias": ((d,), 0.0, 0.02),
            p + "mlp.c_fc.weight": ((d, ff), 0.0, 0.02), p + "mlp.c_fc.bias": ((ff,), 0.0, 0.01),
            p + "mlp.c_proj.weight": ((ff, d), 0.0, proj_std), p + "mlp.c_proj.bias": ((d,), 0.0, 0.01),
        })
    return {name: (mean + std * counter_normal(seed, name, int(np.prod(shape)))).astype(np.float32).reshape(shape)
            for name, (shape, mean, std) in recipe.items()}

"""The plain implementation, pinned by what fixes it beside the reference's text: vectors the
reference's own tests hold, special cases that reduce to a numpy routine, and invariants. Each is
chosen so that a plausible mistake fails it."""

import math
import os

import numpy as np
import pytest

import plain_gpt2 as P
from conftest import TINY_A, TINY_B, random_tokens


def test_layernorm_reference_vector():
    # engine/tests/test_layernorm.c:4-18
    x = np.array([[1.0, 2.0, 3.0], [2.0, 4.0, 6.0]])
    y = P.layernorm(x, np.ones(3), np.zeros(3), 1e-5)
    np.testing.assert_allclose(y, [[-1.2247449, 0, 1.2247449]] * 2, atol=1e-5)


def test_layernorm_invariants():
    rng = np.random.default_rng(0)
    x = rng.standard_normal((5, 37)) * 3 + 1000.0  # a large mean: needs the centred variance
    g, b = rng.standard_normal(37), rng.standard_normal(37)
    y = P.layernorm(x, np.ones(37), np.zeros(37), 1e-5)
    np.testing.assert_allclose(y.mean(-1), 0, atol=1e-9)
    np.testing.assert_allclose(y.var(-1), 1, atol=1e-4)
    # the numpy special case; a biased variance (ddof 0) and eps inside the root
    ref = (x - x.mean(-1, keepdims=True)) / np.sqrt(x.var(-1, keepdims=True) + 1e-5) * g + b
    np.testing.assert_allclose(P.layernorm(x, g, b, 1e-5), ref, rtol=1e-10, atol=1e-9)
    # a constant row gives beta (engine/tests/test_layernorm.cu:176-191)
    np.testing.assert_allclose(P.layernorm(np.full((1, 37), 7.0), g, b, 1e-5), b[None], atol=1e-12)
    # rows are independent
    np.testing.assert_allclose(P.layernorm(x[2:3], g, b, 1e-5), P.layernorm(x, g, b, 1e-5)[2:3])
    # eps matters where the variance is small
    small = rng.standard_normal((1, 37)) * 1e-3
    assert not np.allclose(P.layernorm(small, g, b, 1e-5), P.layernorm(small, g, b, 1e-6))


def test_linear_reference_vector():
    # engine/tests/test_linear.c:4-23 : Conv1D layout [in, out], used without a transpose
    x = np.array([[1.0, 2, 3], [4, 5, 6]])
    w = np.array([[7.0, 8], [9, 10], [11, 12]])
    np.testing.assert_allclose(P.linear(x, w, np.array([1.0, -2])), [[59, 62], [140, 152]])
    np.testing.assert_allclose(P.linear(x, w, None), [[58, 64], [139, 154]])  # test_matrix_mult.c:4-22


def test_embedding_reference_vector():
    # engine/tests/test_embedding.c:4-23
    wte = np.array([[10.0, 11, 12], [20, 21, 22], [30, 31, 32]])
    wpe = np.array([[1.0, 2, 3], [4, 5, 6]])
    np.testing.assert_allclose(P.embed([2, 0], wte, wpe), [[31, 33, 35], [14, 16, 18]])
    np.testing.assert_allclose(P.embed([0], wte, wpe, first_position=1), [[14, 16, 18]])


def test_softmax_reference_vectors():
    # engine/tests/test_softmax.c:4-44
    np.testing.assert_allclose(
        P.softmax(np.array([[1.0, 2, 3], [0, 0, 0]])),
        [[0.0900306, 0.2447285, 0.6652409], [1 / 3] * 3],
        atol=1e-6,
    )
    assert np.isfinite(P.softmax(np.array([[1000.0, 1001, 1002]]))).all()
    np.testing.assert_allclose(
        P.causal_softmax(np.array([[1.0, 2, 3]] * 3)),
        [[1, 0, 0], [0.2689414, 0.7310586, 0], [0.0900306, 0.2447285, 0.6652409]],
        atol=1e-6,
    )


def test_attention_reference_vectors():
    # engine/tests/test_attention.c:4-22 : uniform scores give running means (causal mask)
    ones = np.ones((3, 2))
    v = np.array([[1.0, 10], [3, 20], [5, 30]])
    np.testing.assert_allclose(P.attention_head(ones, ones, v), [[1, 10], [2, 15], [3, 20]], atol=1e-9)
    # engine/tests/test_attention.c:24-54 : fails without the 1/sqrt(head_size) scale
    q = np.array([[1.0, 0], [1, 0]])
    k = np.array([[1.0, 0], [0, 1]])
    v = np.array([[10.0, 1], [0, 20]])
    np.testing.assert_allclose(P.attention_head(q, k, v), [[10, 1], [6.6976156, 7.2745287]], atol=1e-5)


def test_multi_head_reference_vector():
    # engine/tests/test_multi_head_attention.c:4-22 : heads are column blocks, concatenated back
    ones = np.ones((3, 4))
    v = np.array([[1.0, 10, 100, 1000], [3, 20, 300, 2000], [5, 30, 500, 3000]])
    np.testing.assert_allclose(
        P.multi_head_attention(ones, ones, v, 2),
        [[1, 10, 100, 1000], [2, 15, 200, 1500], [3, 20, 300, 2000]],
        atol=1e-9,
    )


def test_attention_last_row_is_plain_softmax_attention():
    # the last row sees every key: it reduces to unmasked softmax(q k^T / sqrt(hs)) v
    rng = np.random.default_rng(1)
    q, k, v = (rng.standard_normal((9, 8)) for _ in range(3))
    s = q[-1] @ k.T / math.sqrt(8)
    p = np.exp(s - s.max())
    np.testing.assert_allclose(P.attention_head(q, k, v)[-1], (p / p.sum()) @ v, rtol=1e-12)
    # causality: a row does not depend on later keys
    np.testing.assert_allclose(P.attention_head(q[:4], k[:4], v[:4]), P.attention_head(q, k, v)[:4], rtol=1e-12)
    # a window of 1 returns the value itself; a window as long as the sequence changes nothing
    np.testing.assert_allclose(P.attention_head(q, k, v, window=1), v, rtol=1e-12)
    np.testing.assert_allclose(P.attention_head(q, k, v, window=9), P.attention_head(q, k, v), rtol=1e-12)


def test_grouped_heads_reduce_to_repeated_heads():
    rng = np.random.default_rng(2)
    q = rng.standard_normal((6, 16))
    k, v = rng.standard_normal((6, 8)), rng.standard_normal((6, 8))
    rep = lambda t: np.concatenate([t[:, :4], t[:, :4], t[:, 4:], t[:, 4:]], axis=1)
    np.testing.assert_allclose(
        P.multi_head_attention(q, k, v, 4, n_kv_head=2), P.multi_head_attention(q, rep(k), rep(v), 4), rtol=1e-12
    )


def test_gelu_vectors():
    # engine/tests/test_gelu.c:6-17 (erf form)
    np.testing.assert_allclose(P.gelu_erf(np.array([0.0, 1.0, 10.0])), [0, 0.8413447, 10], atol=1e-6)
    # tanh form against the formula with sqrt(2/pi) (engine/tests/test_gelu.cu:28-53)
    x = np.array([-6.0, -3, -1, -0.5, 0, 0.5, 1, 3, 6])
    ref = 0.5 * x * (1 + np.tanh(math.sqrt(2 / math.pi) * (x + 0.044715 * x**3)))
    np.testing.assert_allclose(P.gelu_new(x), ref, atol=1e-9)
    assert abs(P.gelu_new(np.array([1.0]))[0] - P.gelu_erf(np.array([1.0]))[0]) > 1e-4  # two functions


def _block_weights(d, ff, rng=None, zero=True):
    z = lambda *s: np.zeros(s)
    return {
        "ln_1.weight": np.ones(d), "ln_1.bias": z(d),
        "attn.c_attn.weight": z(d, 3 * d), "attn.c_attn.bias": z(3 * d),
        "attn.c_proj.weight": z(d, d), "attn.c_proj.bias": z(d),
        "ln_2.weight": np.ones(d), "ln_2.bias": z(d),
        "mlp.c_fc.weight": z(d, ff), "mlp.c_fc.bias": z(ff),
        "mlp.c_proj.weight": z(ff, d), "mlp.c_proj.bias": z(d),
    }


def test_block_reference_vectors():
    # engine/tests/test_transformer_block.c:4-39 : zero projections leave the input
    x = np.arange(1.0, 9.0).reshape(2, 4)
    np.testing.assert_allclose(P.block(x, _block_weights(4, 6), 2, 1e-5, "gelu_new"), x, atol=1e-12)
    # engine/tests/test_transformer_block.c:41-74 : LN -> gelu_new(+-1) added to the residual;
    # fails if the norm stands after the MLP or the residual is taken from the normed input
    w = _block_weights(2, 2)
    w["mlp.c_fc.weight"] = np.eye(2)
    w["mlp.c_proj.weight"] = np.eye(2)
    y = P.block(np.array([[0.0, 2.0]]), w, 1, 1e-5, "gelu_new")
    np.testing.assert_allclose(y, [[-0.1588080, 2.8411920]], atol=1e-5)


def test_qkv_column_order():
    # q, k, v are columns [0,d), [d,2d), [2d,3d) of c_attn (engine/src/gpt2.c:79-90): with only the
    # v columns and c_proj the identity the block adds the running mean of ln_1(x) to x.
    d = 4
    w = _block_weights(d, 2)
    w["attn.c_attn.weight"][:, 2 * d :] = np.eye(d)
    w["attn.c_proj.weight"] = np.eye(d)
    rng = np.random.default_rng(3)
    x = rng.standard_normal((5, d))
    ln = P.layernorm(x, np.ones(d), np.zeros(d), 1e-5)
    running_mean = np.cumsum(ln, axis=0) / np.arange(1, 6)[:, None]
    np.testing.assert_allclose(P.block(x, w, 2, 1e-5, "gelu_new"), x + running_mean, atol=1e-12)


def test_query_and_key_columns_are_not_interchangeable():
    # The reference's own attention vector (engine/tests/test_attention.c:24-54: q = [[1,0],[1,0]],
    # k = [[1,0],[0,1]], v = [[10,1],[0,20]] -> second row [6.6976156, 7.2745287]) routed through the
    # whole block, so that it fixes WHICH columns of c_attn are q and which are k
    # (engine/src/gpt2.c:79-90: q = [0,d), k = [d,2d)). With the two swapped the second row's scores
    # are equal and it comes out as the mean of v, [5, 10.5].
    d = 2
    w = _block_weights(d, 2)
    x = np.eye(2)                                    # ln_1(x) = [[1,-1],[-1,1]] (eps next to nothing)
    w["attn.c_attn.bias"][0:2] = [1.0, 0.0]          # q: the bias alone, the same in both rows
    w["attn.c_attn.weight"][:, 2:4] = [[0.25, -0.25], [-0.25, 0.25]]
    w["attn.c_attn.bias"][2:4] = [0.5, 0.5]          # k = [[1,0],[0,1]]
    w["attn.c_attn.weight"][:, 4:6] = [[5.0, -9.5], [0.0, 0.0]]
    w["attn.c_attn.bias"][4:6] = [5.0, 10.5]         # v = [[10,1],[0,20]]
    w["attn.c_proj.weight"] = np.eye(d)
    y = P.block(x, w, 1, 1e-14, "gelu_new")
    np.testing.assert_allclose(y - x, [[10.0, 1.0], [6.6976156, 7.2745287]], atol=2e-6)
    assert np.abs((y - x)[1] - [5.0, 10.5]).max() > 1.0


def test_model_reduces_to_embedding_head_when_blocks_are_zero():
    cfg = dict(TINY_A, n_inner=256)
    w = P.random_weights(cfg, 0)
    for name in w:
        if name.startswith("h.") and ("c_attn" in name or "c_proj" in name or "c_fc" in name):
            w[name] = np.zeros_like(w[name])
    toks = random_tokens(1, 11, cfg["vocab_size"])
    h = w["wte.weight"][toks].astype(np.float64) + w["wpe.weight"][: len(toks)]
    ref = P.layernorm(h, w["ln_f.weight"].astype(np.float64), w["ln_f.bias"], 1e-5) @ w["wte.weight"].T.astype(np.float64)
    np.testing.assert_allclose(P.forward(cfg, w, toks), ref, rtol=1e-10, atol=1e-12)


@pytest.mark.parametrize("cfg,seed", [(dict(TINY_A, n_inner=256), 0), (TINY_B, 2)])
def test_model_causality_and_options(cfg, seed):
    w = P.random_weights(cfg, seed)
    toks = random_tokens(5, 20, cfg["vocab_size"])
    full = P.forward(cfg, w, toks)
    assert full.shape == (20, cfg["vocab_size"])
    # logits at t do not depend on later tokens
    np.testing.assert_allclose(P.forward(cfg, w, toks[:7]), full[:7], rtol=1e-9, atol=1e-12)
    # the activation switch and eps are really used
    other = "gelu" if cfg["activation_function"] == "gelu_new" else "gelu_new"
    assert np.abs(P.forward(dict(cfg, activation_function=other), w, toks) - full).max() > 1e-6
    assert np.abs(P.forward(dict(cfg, layer_norm_epsilon=1e-2), w, toks) - full).max() > 1e-6
    # float32 arithmetic stays close to float64
    assert np.abs(P.forward(cfg, w, toks, dtype=np.float32) - full).max() < 1e-4


def test_top_p_keep():
    p = np.array([0.5, 0.2, 0.2, 0.05, 0.05])
    assert P.top_p_keep(p, 0.6).tolist() == [True, True, True, False, False]
    assert P.top_p_keep(p, 0.5).tolist() == [True, False, False, False, False]
    assert P.top_p_keep(p, 1.0).tolist() == [True] * 5


def test_safetensors_roundtrip(tmp_path):
    w = P.random_weights(dict(TINY_B), 2)
    P.write_safetensors(tmp_path / "m.safetensors", w)
    back = P.read_safetensors(tmp_path / "m.safetensors")
    assert back.keys() == w.keys() and all((back[k] == w[k]).all() for k in w)
    P.write_safetensors(tmp_path / "b.safetensors", w, bf16=True)
    back = P.read_safetensors(tmp_path / "b.safetensors")
    np.testing.assert_array_equal(back["wte.weight"], P.round_to_bf16(w["wte.weight"]))
    # round to nearest even, checked on hand-picked bit patterns
    x = np.array([0x3F808000, 0x3F818000, 0x3F808001], dtype=np.uint32).view(np.float32)
    assert P.f32_to_bf16_rne(x).tolist() == [0x3F80, 0x3F82, 0x3F81]


# The reference repository's root, where a checkout of it is at hand (MINI_LLM_REFERENCE=/path/to/mini_llm).
REFERENCE_DUMPS = os.path.join(os.environ.get("MINI_LLM_REFERENCE", ""), "engine", "tests", "reference_data")


@pytest.mark.skipif(not os.environ.get("MINI_LLM_REFERENCE") or not os.path.isdir(REFERENCE_DUMPS),
                    reason="MINI_LLM_REFERENCE does not name a checkout of the reference with its dumped activations")
def test_dumped_activations_of_the_real_model_follow_the_plain_formulas():
    # The reference holds what every part of the real GPT-2 put out for the tokens 15496, 11, 995
    # (scripts/dump_reference.py:76-140: the three gathered embedding rows, per block the outputs of
    # ln_1, attention, ln_2, the feed-forward and the block, ln_f, all logits), but not the weights.
    # What they fix without the weights: the embedding is the sum of the two rows; a block is
    # x + attention + feed-forward; ln_1 reads the block's input, ln_2 the sum after attention, ln_f
    # the last block (a norm's output is gain * normalised + offset per column, so over the three
    # rows the points (normalised, output) of a column lie on one line, and only for the right
    # input); the head is the token table again, without a bias; the next token is the argmax.
    def dump(name, shape=(3, 768)):
        return np.fromfile(f"{REFERENCE_DUMPS}/{name}.bin", dtype="<f4").reshape(shape).astype(np.float64)

    def off_the_line(x, y):
        normalised = P.layernorm(x, np.ones(x.shape[1]), np.zeros(x.shape[1]), 1e-5)
        gain = (y[1] - y[0]) / (normalised[1] - normalised[0])
        return np.abs(gain * (normalised[2] - normalised[0]) + y[0] - y[2]).max()

    token_rows, position_rows = dump("wte"), dump("wpe")
    x = P.embed([0, 1, 2], token_rows, position_rows)
    for layer in range(12):
        name = f"block_{layer:02d}"
        attention, mlp, out = dump(name + "_attn"), dump(name + "_mlp"), dump(name)
        np.testing.assert_allclose(x + attention + mlp, out, rtol=0, atol=5e-4)
        assert off_the_line(x, dump(name + "_ln1")) < 1e-4
        assert off_the_line(x + attention, dump(name + "_ln2")) < 1e-4
        assert off_the_line(x, dump(name + "_ln2")) > 1.0  # the norm in the wrong place shows
        x = out
    final = dump("ln_f")
    assert off_the_line(x, final) < 1e-3   # outputs up to 180 here
    logits = dump("logits_full", (3, 50257))
    np.testing.assert_allclose(P.lm_head(final, token_rows), logits[:, [15496, 11, 995]], rtol=0, atol=1e-4)
    np.testing.assert_array_equal(dump("logits_last", (50257,)), logits[2])
    with open(f"{REFERENCE_DUMPS}/expected_next_token.txt") as f:
        assert int(logits[2].argmax()) == int(f.read()) == 13

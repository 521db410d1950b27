"""Weights by name: one error that lists everything wrong, dtype and layout handling, and the
random-weights mode."""

import json

import numpy as np
import pytest
import torch

import plain_gpt2
from conftest import TINY_A, TINY_B, make_plain_model_dir
from mini_llm_amd.config import config_from_dict, get_architecture
from mini_llm_amd.precision import Precision
from mini_llm_amd.weights import SafetensorsFile, WeightsError, load_weights, write_model_dir, write_safetensors


def build(config_dict, dtype="float32"):
    config = config_from_dict(config_dict)
    return get_architecture(config.architecture).build(config, Precision.from_name(dtype))


def write(folder, tensors):
    write_safetensors(folder / "model.safetensors", {k: torch.as_tensor(v) for k, v in tensors.items()})


def test_loads_by_name_with_or_without_prefix(tmp_path):
    for prefix in ("transformer.", ""):
        folder = tmp_path / f"p{len(prefix)}"
        weights = make_plain_model_dir(folder, TINY_B, 2, prefix=prefix)
        model = build(TINY_B)
        load_weights(model, folder, "cpu")
        # Conv1D [in, out] in the file, kept [out, in]
        kept = model.blocks[1].mixer.qkv.weight
        assert kept.shape == (288, 96) and kept.dtype == torch.float32 and kept.is_contiguous()
        np.testing.assert_array_equal(kept.numpy(), weights["h.1.attn.c_attn.weight"].T)
        np.testing.assert_array_equal(model.embedding.weight.numpy(), weights["wte.weight"])
        np.testing.assert_array_equal(model.blocks[2].norm_2.bias.numpy(), weights["h.2.ln_2.bias"])
        np.testing.assert_array_equal(model.final_norm.weight.numpy(), weights["ln_f.weight"])


def test_masks_and_tied_head_in_the_file_are_ignored(tmp_path):
    weights = plain_gpt2.random_weights(dict(TINY_A, n_inner=256), 0)
    extra = dict(weights)
    extra["h.0.attn.bias"] = np.ones((1, 1, 128, 128), dtype=np.float32)
    extra["h.1.attn.masked_bias"] = np.float32(-1e4).reshape(())
    extra["lm_head.weight"] = weights["wte.weight"]
    write(tmp_path, {"transformer." + k if k != "lm_head.weight" else k: v for k, v in extra.items()})
    load_weights(build(TINY_A), tmp_path, "cpu")


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    weights = plain_gpt2.random_weights(dict(TINY_A, n_inner=256), 0)
    del weights["h.1.mlp.c_fc.bias"], weights["ln_f.weight"]
    weights["h.0.attn.c_proj.weight"] = np.zeros((64, 65), dtype=np.float32)
    weights["wpe.weight"] = weights["wpe.weight"][:100]
    weights["h.7.ln_1.weight"] = np.zeros(64, dtype=np.float32)
    weights["score.weight"] = np.zeros((2, 64), dtype=np.float32)
    write(tmp_path, weights)
    with pytest.raises(WeightsError) as info:
        load_weights(build(TINY_A), tmp_path, "cpu")
    e = info.value
    assert e.missing == ["h.1.mlp.c_fc.bias", "ln_f.weight"]
    assert e.unexpected == ["h.7.ln_1.weight", "score.weight"]
    assert [(n, got, want) for n, got, want in e.wrong_shape] == [
        ("h.0.attn.c_proj.weight", (64, 65), (64, 64)), ("wpe.weight", (100, 64), (128, 64))]
    text = str(e)
    for word in ("h.1.mlp.c_fc.bias", "ln_f.weight", "h.7.ln_1.weight", "score.weight", "[64, 65]", "expected [128, 64]"):
        assert word in text


def test_a_transposed_matrix_is_a_wrong_shape(tmp_path):
    weights = plain_gpt2.random_weights(TINY_B, 2)
    weights["h.0.mlp.c_fc.weight"] = weights["h.0.mlp.c_fc.weight"].T.copy()  # [out, in]: not GPT-2's layout
    write(tmp_path, weights)
    with pytest.raises(WeightsError, match=r"h.0.mlp.c_fc.weight is \[320, 96\], expected \[96, 320\]"):
        load_weights(build(TINY_B), tmp_path, "cpu")


def test_broken_files(tmp_path):
    with pytest.raises(WeightsError, match="does not exist"):
        load_weights(build(TINY_A), tmp_path, "cpu")
    make_plain_model_dir(tmp_path, TINY_A, 0)
    raw = (tmp_path / "model.safetensors").read_bytes()
    (tmp_path / "model.safetensors").write_bytes(raw[: len(raw) // 2])
    with pytest.raises(WeightsError, match="truncated"):
        load_weights(build(TINY_A), tmp_path, "cpu")
    (tmp_path / "model.safetensors").write_bytes(b"\x10\x00\x00\x00\x00\x00\x00\x00{not json at all}")
    with pytest.raises(WeightsError, match="not valid JSON"):
        load_weights(build(TINY_A), tmp_path, "cpu")
    (tmp_path / "model.safetensors").write_bytes(b"\xff" * 8 + b"{}")
    with pytest.raises(WeightsError, match="exceeds the file"):
        load_weights(build(TINY_A), tmp_path, "cpu")


def test_integer_tensor_where_floats_belong(tmp_path):
    weights = plain_gpt2.random_weights(dict(TINY_A, n_inner=256), 0)
    weights["ln_f.bias"] = np.zeros(64, dtype=np.int32)
    write(tmp_path, weights)
    with pytest.raises(WeightsError, match="ln_f.bias holds integers"):
        load_weights(build(TINY_A), tmp_path, "cpu")


@pytest.mark.parametrize("stored_bf16", [False, True])
@pytest.mark.parametrize("run", ["float32", "bfloat16"])
def test_element_types_kept(tmp_path, stored_bf16, run):
    weights = make_plain_model_dir(tmp_path, TINY_B, 2, bf16=stored_bf16)
    model = build(TINY_B, run)
    load_weights(model, tmp_path, "cpu")
    matrix, table, vector = model.blocks[0].feed_forward.up.weight, model.embedding.weight, model.blocks[0].norm_1.weight
    want = torch.float32 if run == "float32" else torch.bfloat16
    assert matrix.dtype == want and table.dtype == want and model.position_encoding.weight.dtype == want
    assert vector.dtype == torch.float32 and model.blocks[0].feed_forward.up.bias.dtype == torch.float32
    ref = weights["h.0.ln_1.weight"]
    if stored_bf16:
        ref = plain_gpt2.round_to_bf16(ref)
    np.testing.assert_array_equal(vector.numpy(), ref)  # a vector stored in 32-bit stays exactly so
    ref = weights["wte.weight"]
    if stored_bf16 or run == "bfloat16":
        ref = plain_gpt2.round_to_bf16(ref)
    np.testing.assert_array_equal(table.float().numpy(), ref)


def test_random_weights_mode_writes_a_folder_the_loader_reads(tmp_path):
    config = config_from_dict(TINY_B)
    write_model_dir(config, 7, tmp_path / "m")
    assert config_from_dict(json.loads((tmp_path / "m" / "config.json").read_text())) == config
    model = build(TINY_B)
    load_weights(model, tmp_path / "m", "cpu")
    # the plain reader sees the same numbers under the reference's tensor names
    _, plain = plain_gpt2.load_model_dir(tmp_path / "m")
    np.testing.assert_array_equal(model.blocks[2].feed_forward.down.weight.numpy(), plain["h.2.mlp.c_proj.weight"].T)
    # the recipe: standard deviations by role
    L = config.n_layer
    assert abs(plain["wte.weight"].std() - 0.02) < 1e-3
    assert abs(plain["h.0.attn.c_attn.weight"].std() - 0.02) < 1e-3
    assert abs(plain["h.1.attn.c_proj.weight"].std() - 0.02 / np.sqrt(2 * L)) < 5e-4
    assert abs(plain["h.1.mlp.c_proj.weight"].std() - 0.02 / np.sqrt(2 * L)) < 5e-4
    assert abs(plain["h.0.mlp.c_fc.bias"].std() - 0.01) < 2e-3
    assert abs(plain["ln_f.weight"].mean() - 1.0) < 2e-2 and abs(plain["ln_f.weight"].std() - 0.05) < 1.5e-2
    assert abs(plain["h.2.ln_2.bias"].std() - 0.02) < 6e-3
    # the seed decides: same seed same file, another seed other numbers
    write_model_dir(config, 7, tmp_path / "again")
    write_model_dir(config, 8, tmp_path / "other")
    assert (tmp_path / "again" / "model.safetensors").read_bytes() == (tmp_path / "m" / "model.safetensors").read_bytes()
    assert (tmp_path / "other" / "model.safetensors").read_bytes() != (tmp_path / "m" / "model.safetensors").read_bytes()
    # stored in bfloat16 on request
    write_model_dir(config, 7, tmp_path / "bf", dtype="bfloat16")
    f = SafetensorsFile(tmp_path / "bf" / "model.safetensors")
    assert f.dtype("wte.weight") == torch.bfloat16 and f.shape("wte.weight") == (1000, 96)


def test_random_weights_are_the_documented_counter_based_draws(tmp_path):
    """Every element is a function of (seed, tensor name, element index): the framework's folder
    equals, bit for bit, what the plain implementation's own copy of the generator draws; a
    tensor's numbers do not depend on its shape's split, and a few values are pinned."""
    from mini_llm_amd.weights.counter_rng import normal_tensor, tensor_key

    for raw, seed in ((TINY_A, 0), (TINY_B, 7)):
        folder = tmp_path / f"m{seed}"
        write_model_dir(config_from_dict(raw), seed, folder)
        _, written = plain_gpt2.load_model_dir(folder)
        twin = plain_gpt2.counter_random_weights(raw, seed)
        assert sorted(written) == sorted(twin)
        for name in twin:
            assert written[name].dtype == np.float32
            np.testing.assert_array_equal(written[name], twin[name], err_msg=name)
    # element i is the same whether asked for alone, in a longer tensor, or across a chunk border
    long = normal_tensor(3, "t", (300_000,))
    np.testing.assert_array_equal(long[:7], normal_tensor(3, "t", (7,)))
    np.testing.assert_array_equal(long.reshape(3, 100_000)[2], long[200_000:])
    np.testing.assert_array_equal(long[131_070:131_075], plain_gpt2.counter_normal(3, "t", 131_075)[131_070:].astype(np.float32))
    # name and seed both decide
    assert not np.array_equal(long[:7], normal_tensor(3, "u", (7,))) and not np.array_equal(long[:7], normal_tensor(4, "t", (7,)))
    # pinned: the integer part exactly, the values to the last bit of float32
    assert tensor_key(5, "wte.weight") == plain_key(5, "wte.weight") == 0xF103BFA14EA3A977
    bits = lambda *a: [int(v) for v in normal_tensor(*a).view(np.uint32)]
    assert bits(5, "wte.weight", (4,), 0.0, 0.02) == [0xBC4D3DD8, 0x3C783C2F, 0x3CBA8C95, 0xBBFEB98D]   # -0.0125269, 0.0151511, 0.0227721, -0.0077736
    assert bits(0, "ln_f.bias", (4,), 1.0, 0.05) == [0x3F70A79D, 0x3F866C6B, 0x3F82D16B, 0x3F89BB6E]    # 0.9400576, 1.0501837, 1.0220159, 1.0760324
    draws = normal_tensor(11, "h.0.mlp.c_fc.weight", (1000, 1000))
    assert abs(draws.mean()) < 3e-3 and abs(draws.std() - 1.0) < 3e-3 and abs((draws**4).mean() - 3.0) < 0.05   # normal, not merely centred


def plain_key(seed, name):
    m = (1 << 64) - 1
    h = 0xCBF29CE484222325
    for byte in name.encode():
        h = ((h ^ byte) * 0x100000001B3) & m
    def mix(z):
        z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & m
        z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & m
        return z ^ (z >> 31)
    return mix(mix(seed & m) ^ h)

"""Weights: reading by name, the one error that lists every misfit, precision rules, random folders."""
import json
import struct

import pytest
import torch

from geneinfer_amd.config import parse_config
from geneinfer_amd.parts import model_tensor_needs
from geneinfer_amd.weights import (SafetensorsError, SafetensorsFile, TensorNeed, WeightsError, load_tensors, random_tensors,
                                   write_random_model, write_safetensors)
from model_folders import CONFIGS, full_config, random_weights, tensor_layout, write_model, write_safetensors_by_hand
from plain_llama import read_model_folder


def needs_of(name):
    spec = parse_config(full_config(CONFIGS[name])).model_spec()
    return spec, model_tensor_needs(spec)


@pytest.mark.parametrize("name", ["A", "B"])
def test_the_model_asks_for_exactly_the_reference_layout(name):
    spec, needs = needs_of(name)
    want = dict(tensor_layout(full_config(CONFIGS[name])))            # src/loader/hf_checkpoint.cpp:214-235
    got = {n.name: n.shape for n in needs}
    assert got == want
    assert all(n.role == "norm" for n in needs if n.name.endswith("norm.weight"))


def test_loading_by_name_from_a_shuffled_file(tmp_path):
    w = write_model(tmp_path, CONFIGS["B"], seed=4, dtype=torch.bfloat16, norm_dtype=torch.float32)
    spec, needs = needs_of("B")
    t = load_tensors(tmp_path, needs, torch.bfloat16, "cpu", spec.ignorable_tensors)
    for name, src in w.items():
        if name.endswith("norm.weight"):
            assert t[name].dtype == torch.float32 and torch.equal(t[name], src)          # stored in 32-bit: stays so
        else:
            assert t[name].dtype == torch.bfloat16 and torch.equal(t[name], src.to(torch.bfloat16))
    wide = load_tensors(tmp_path, needs, torch.float32, "cpu", spec.ignorable_tensors)
    assert all(v.dtype == torch.float32 for v in wide.values())
    name = "model.layers.1.mlp.up_proj.weight"
    assert torch.equal(wide[name], w[name].to(torch.bfloat16).float())                   # widened exactly


def test_float32_file_stays_float32_and_float16_is_widened(tmp_path):
    spec, needs = needs_of("A")
    write_model(tmp_path / "f32", CONFIGS["A"], seed=1, dtype=torch.float32)
    assert all(v.dtype == torch.float32 for v in load_tensors(tmp_path / "f32", needs, torch.bfloat16, "cpu", spec.ignorable_tensors).values())
    w = write_model(tmp_path / "f16", CONFIGS["A"], seed=1, dtype=torch.float16)
    t = load_tensors(tmp_path / "f16", needs, torch.bfloat16, "cpu", spec.ignorable_tensors)
    name = "model.layers.0.self_attn.q_proj.weight"
    assert t[name].dtype == torch.float32 and torch.equal(t[name], w[name].half().float())


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    cfg = full_config(CONFIGS["B"])
    w = random_weights(cfg, 0)
    del w["model.layers.2.mlp.down_proj.weight"], w["model.norm.weight"]
    w["model.layers.0.self_attn.k_proj.weight"] = torch.zeros(7, 96)
    w["model.embed_tokens.weight"] = torch.zeros(384, 95)
    w["model.layers.9.extra.weight"] = torch.zeros(3)
    w["lm_head.weight"] = torch.zeros(384, 96, dtype=torch.int32)
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    write_safetensors_by_hand(tmp_path / "model.safetensors", w, shuffle_seed=3)
    spec, needs = needs_of("B")
    with pytest.raises(WeightsError) as e:
        load_tensors(tmp_path, needs, torch.bfloat16, "cpu", spec.ignorable_tensors)
    msg = str(e.value)
    assert "missing tensors (2)" in msg and "model.layers.2.mlp.down_proj.weight" in msg and "model.norm.weight" in msg
    assert "unexpected tensors (1)" in msg and "model.layers.9.extra.weight" in msg
    assert "wrong shapes (2)" in msg and "file has [7, 96], the model needs [32, 96]" in msg and "file has [384, 95]" in msg
    assert "unsupported dtypes (1)" in msg and "lm_head.weight: I32" in msg


def test_tensors_a_model_may_ignore(tmp_path):
    cfg = full_config(CONFIGS["A"])                                    # tied: a stray lm_head and rotary tables are not errors
    w = random_weights(cfg, 2)
    w["lm_head.weight"] = torch.ones(256, 64)
    w["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.ones(8)
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    write_safetensors_by_hand(tmp_path / "model.safetensors", w)
    spec, needs = needs_of("A")
    t = load_tensors(tmp_path, needs, torch.float32, "cpu", spec.ignorable_tensors)
    assert "lm_head.weight" not in t and torch.equal(t["model.embed_tokens.weight"], w["model.embed_tokens.weight"])


def test_missing_files_and_sharded_checkpoints(tmp_path):
    spec, needs = needs_of("A")
    with pytest.raises(WeightsError, match="no model.safetensors"):
        load_tensors(tmp_path, needs, torch.float32, "cpu")
    (tmp_path / "model.safetensors.index.json").write_text("{}")
    with pytest.raises(WeightsError, match="sharded"):
        load_tensors(tmp_path, needs, torch.float32, "cpu")


def test_integer_tables_become_int32_and_odd_alignment_is_read(tmp_path):
    tensors = {"table": torch.arange(6, dtype=torch.int64).reshape(2, 3), "w": torch.randn(3, 5).to(torch.bfloat16)}
    write_safetensors_by_hand(tmp_path / "model.safetensors", tensors, header_pad=1)   # data at odd addresses
    t = load_tensors(tmp_path, [TensorNeed("table", (2, 3), "table"), TensorNeed("w", (3, 5))], torch.bfloat16, "cpu")
    assert t["table"].dtype == torch.int32 and t["table"].tolist() == [[0, 1, 2], [3, 4, 5]]
    assert torch.equal(t["w"], tensors["w"])


@pytest.mark.parametrize("damage,message", [
    (lambda raw, hlen: raw[:4], "too small"),
    (lambda raw, hlen: struct.pack("<Q", len(raw)) + raw[8:], "does not fit the file"),
    (lambda raw, hlen: raw[:8] + b"[" + raw[9:], "not valid JSON|not a JSON object"),
    (lambda raw, hlen: raw[:len(raw) - 3], "outside the file"),
])
def test_damaged_files_are_refused(tmp_path, damage, message):              # src/loader/safetensors.cpp:25-88
    path = tmp_path / "model.safetensors"
    write_safetensors(path, {"a": torch.ones(4, 4), "b": torch.zeros(8)})
    raw = path.read_bytes()
    (hlen,) = struct.unpack("<Q", raw[:8])
    path.write_bytes(damage(raw, hlen))
    with pytest.raises(SafetensorsError, match=message):
        SafetensorsFile(path)


def test_size_that_does_not_match_the_shape_is_refused(tmp_path):
    header = json.dumps({"a": {"dtype": "F32", "shape": [3], "data_offsets": [0, 8]}}).encode()
    (tmp_path / "m.safetensors").write_bytes(struct.pack("<Q", len(header)) + header + b"\0" * 8)
    with pytest.raises(SafetensorsError, match="holds 8 bytes, its shape needs 12"):
        SafetensorsFile(tmp_path / "m.safetensors")


def test_written_files_read_back(tmp_path):
    tensors = {"x": torch.randn(5, 7), "y": torch.randn(3).to(torch.bfloat16), "z": torch.arange(4, dtype=torch.int32)}
    write_safetensors(tmp_path / "t.safetensors", tensors, metadata={"format": "pt"})
    f = SafetensorsFile(tmp_path / "t.safetensors")
    assert f.metadata == {"format": "pt"} and set(f.entries) == set(tensors)
    for k, v in tensors.items():
        assert torch.equal(f.tensor(k), v)


@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
def test_random_model_folder_is_seeded_and_complete(tmp_path, dtype):
    config = parse_config(full_config(CONFIGS["B"]))
    write_random_model(tmp_path / "a", config, seed=7, dtype=dtype)
    write_random_model(tmp_path / "b", config, seed=7, dtype=dtype)
    write_random_model(tmp_path / "c", config, seed=8, dtype=dtype)
    cfg_a, ta = read_model_folder(tmp_path / "a")                      # the plain reader understands what was written
    _, tb = read_model_folder(tmp_path / "b")
    _, tc = read_model_folder(tmp_path / "c")
    assert parse_config(cfg_a) == config
    assert set(ta) == {n for n, _ in tensor_layout(full_config(CONFIGS["B"]))}
    assert all(torch.equal(ta[k], tb[k]) for k in ta) and not torch.equal(ta["lm_head.weight"], tc["lm_head.weight"])
    q = ta["model.layers.0.self_attn.q_proj.weight"].float()
    assert abs(float(q.std()) - 0.02) < 0.002 and abs(float(q.mean())) < 0.002
    n = ta["model.layers.0.input_layernorm.weight"].float()
    assert abs(float(n.mean()) - 1.0) < 0.05 and 0.05 < float(n.std()) < 0.15
    spec = config.model_spec()
    loaded = load_tensors(tmp_path / "a", model_tensor_needs(spec), torch.bfloat16, "cpu", spec.ignorable_tensors)
    assert set(loaded) == set(ta)


def test_random_tensors_refuse_integer_tables():
    with pytest.raises(ValueError, match="integer tables"):
        random_tensors([TensorNeed("t", (2,), "table")], 0)


def test_the_formula_of_the_weights_drawn_on_the_device_is_the_stated_one():
    """`formula_values` (the product's statement of what the device kernel draws) against this suite's own restatement
    (`model_folders.formula_weights`) and, for three elements, against the formula worked with Python's integers and math."""
    import math
    from geneinfer_amd.weights import formula_values, tensor_key
    from model_folders import TINY_C, formula_weights, full_config, tensor_layout
    cfg = full_config(TINY_C)
    ours = formula_weights(cfg, seed=11, std=0.03)
    for name, shape in tensor_layout(cfg):
        offset, scale = (1.0, 0.1) if name.endswith("norm.weight") else (0.0, 0.03)
        assert torch.equal(formula_values(name, shape, 11, offset, scale), ours[name]), name
    name, golden, mask = "model.layers.0.mlp.up_proj.weight", 0x9E3779B97F4A7C15, (1 << 64) - 1
    key = 0xCBF29CE484222325
    for byte in name.encode():
        key = ((key ^ byte) * 0x100000001B3) & mask
    key = (key + 12 * golden) & mask
    assert key == tensor_key(name, 11)
    flat = ours[name].reshape(-1)
    for i in (0, 1, 4000):
        z = (key + (i + 1) * golden) & mask
        z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & mask
        z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & mask
        z ^= z >> 31
        u1, u2 = ((z >> 40) + 1) / 2 ** 24, ((z >> 8) & 0xFFFFFF) / 2 ** 24
        want = 0.03 * math.sqrt(-2.0 * math.log(u1)) * math.cos(2.0 * math.pi * u2)
        assert abs(float(flat[i]) - want) <= 1e-9 + 1e-7 * abs(want)
    every = torch.cat([t.reshape(-1) for n, t in ours.items() if not n.endswith("norm.weight")])
    assert abs(float(every.mean())) < 3e-4 and abs(float(every.std()) - 0.03) < 3e-4               # N(0, std)

"""Safetensors reading/writing, the one weight error, storage types and random weights (CPU)."""
import json
import os
import struct

import pytest
import torch

from conftest import TINY_A, TINY_B
from pulse_infer_amd.config import Qwen3Config
from pulse_infer_amd.models.causal_lm import expected_tensors
from pulse_infer_amd.weights import (DictSource, RandomSource, SafetensorsError, SafetensorsFile, SafetensorsSource,
                                     TensorSpec, WeightError, WeightLoader, check, storage_dtype, write_model_folder,
                                     write_safetensors)


def _raw_file(path, header: dict, payload: bytes = b""):
    blob = json.dumps(header).encode()
    with open(path, "wb") as fh:
        fh.write(struct.pack("<Q", len(blob)) + blob + payload)


def test_round_trip_and_agreement_with_the_safetensors_package(tmp_path):
    from safetensors.torch import load_file, save_file

    tensors = {"a": torch.randn(3, 5).to(torch.bfloat16), "b": torch.randn(7), "c": torch.arange(6, dtype=torch.int32).view(2, 3)}
    ours = str(tmp_path / "ours.safetensors")
    write_safetensors(ours, tensors, metadata={"format": "pt"})
    theirs = load_file(ours)
    f = SafetensorsFile(ours)
    assert f.metadata == {"format": "pt"} and sorted(f.names()) == ["a", "b", "c"]
    for name, t in tensors.items():
        assert torch.equal(theirs[name], t) and torch.equal(f.get(name), t)
        assert f.info(name).dtype == t.dtype and f.info(name).shape == tuple(t.shape)
    lib = str(tmp_path / "lib.safetensors")
    save_file(tensors, lib)
    g = SafetensorsFile(lib)
    for name, t in tensors.items():
        assert torch.equal(g.get(name), t)


def test_header_checks(tmp_path):
    """The reference's negative cases (tests/core/test_safetensor.cpp:33-49: zero elements, byte size overflow)
    and the other checks of its reader (src/core/safetensor.cpp:283-378)."""
    p = str(tmp_path / "x.safetensors")
    with open(p, "wb") as fh:
        fh.write(b"1234")
    with pytest.raises(SafetensorsError, match="too small"):
        SafetensorsFile(p)
    with open(p, "wb") as fh:
        fh.write(struct.pack("<Q", 1 << 40) + b"{}")
    with pytest.raises(SafetensorsError, match="header size"):
        SafetensorsFile(p)
    with open(p, "wb") as fh:
        fh.write(struct.pack("<Q", 5) + b"{nope")
    with pytest.raises(SafetensorsError, match="JSON"):
        SafetensorsFile(p)
    cases = [
        ({"t": {"dtype": "F32", "shape": [0, 4], "data_offsets": [0, 0]}}, b"", "zero elements"),
        ({"t": {"dtype": "F32", "shape": [2, 2], "data_offsets": [0, 12]}}, b"\0" * 16, "do not match"),
        ({"t": {"dtype": "F32", "shape": [1 << 40, 1 << 40], "data_offsets": [0, 16]}}, b"\0" * 16, "do not match"),
        ({"t": {"dtype": "F32", "shape": [-1, 4], "data_offsets": [0, 16]}}, b"\0" * 16, "negative"),
        ({"t": {"dtype": "F32", "shape": [4], "data_offsets": [8, 4]}}, b"\0" * 16, "begin > end"),
        ({"t": {"dtype": "F32", "shape": [8], "data_offsets": [0, 32]}}, b"\0" * 16, "beyond the payload"),
        ({"t": {"dtype": "F8_E4M3", "shape": [4], "data_offsets": [0, 4]}}, b"\0" * 4, "unsupported dtype"),
        ({"t": {"dtype": "F32", "shape": [4]}}, b"\0" * 16, "data_offsets"),
        ({"a": {"dtype": "F32", "shape": [2], "data_offsets": [0, 8]},
          "b": {"dtype": "F32", "shape": [2], "data_offsets": [4, 12]}}, b"\0" * 16, "overlap"),
        ({"__metadata__": {"k": 3}, "a": {"dtype": "F32", "shape": [2], "data_offsets": [0, 8]}}, b"\0" * 8, "__metadata__"),
    ]
    for header, payload, message in cases:
        _raw_file(p, header, payload)
        with pytest.raises(SafetensorsError, match=message):
            SafetensorsFile(p)


def test_one_error_lists_missing_unexpected_and_wrong_shapes():
    cfg = Qwen3Config.from_dict(TINY_B)
    expected = expected_tensors(cfg.model_spec())
    tensors = {n: torch.zeros(s.shape, dtype=torch.bfloat16) for n, s in expected.items()}
    check(DictSource(tensors), expected)  # complete: no error
    del tensors["model.layers.1.mlp.up_proj.weight"]
    del tensors["model.norm.weight"]
    tensors["model.layers.0.self_attn.q_proj.weight"] = torch.zeros(5, 7)
    tensors["model.layers.2.self_attn.k_norm.weight"] = torch.zeros(33)
    tensors["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(16)
    with pytest.raises(WeightError) as err:
        check(DictSource(tensors, "somewhere"), expected)
    e = err.value
    assert sorted(e.missing) == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"]
    assert e.unexpected == ["model.layers.0.self_attn.rotary_emb.inv_freq"]
    assert sorted(n for n, _, _ in e.wrong_shape) == ["model.layers.0.self_attn.q_proj.weight",
                                                      "model.layers.2.self_attn.k_norm.weight"]
    text = str(e)
    for needle in ("somewhere", "missing tensors (2)", "model.norm.weight", "unexpected tensors (1)", "inv_freq",
                   "wrong shapes (2)", "expected [192, 96], found [5, 7]", "expected [32], found [33]"):
        assert needle in text, needle


def test_tensors_that_no_part_asked_for():
    """Alone they do not fail a load (a warning counts them) unless strict is set; when the load fails anyway the
    error names them, strict or not."""
    cfg = Qwen3Config.from_dict(TINY_B)
    expected = expected_tensors(cfg.model_spec())
    tensors = {n: torch.zeros(s.shape, dtype=torch.bfloat16) for n, s in expected.items()}
    tensors["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(16)
    tensors["extra.bias"] = torch.zeros(3)
    assert check(DictSource(tensors), expected) == ["extra.bias", "model.layers.0.self_attn.rotary_emb.inv_freq"]
    with pytest.warns(UserWarning, match="2 tensors .* belong to no part"):
        loader = WeightLoader(DictSource(tensors, "folder"), expected, "bfloat16", "cpu")
    assert loader.ignored == ["extra.bias", "model.layers.0.self_attn.rotary_emb.inv_freq"]
    with pytest.raises(WeightError, match=r"unexpected tensors \(2\)") as strict:
        check(DictSource(tensors), expected, strict=True)
    assert not strict.value.missing and not strict.value.wrong_shape
    del tensors["model.norm.weight"]
    with pytest.raises(WeightError) as err:
        check(DictSource(tensors), expected)
    assert err.value.missing == ["model.norm.weight"] and len(err.value.unexpected) == 2


def test_float16_is_not_rounded_to_bfloat16_silently():
    expected = {"w": TensorSpec((2, 2)), "v": TensorSpec((2, 2)), "n": TensorSpec((2,), kind="norm")}
    big = torch.tensor([[1.0009765625, 2.0], [3.0, 4.0]], dtype=torch.float16)    # 1 + 2^-10: no bfloat16 value
    src = DictSource({"w": big, "v": torch.ones(2, 2, dtype=torch.bfloat16), "n": torch.ones(2)}, "half")
    with pytest.raises(WeightError, match="would round") as err:
        WeightLoader(src, expected, "bfloat16", "cpu")
    assert err.value.narrowed == [("w", "float16")] and "w (float16)" in str(err.value)
    wide = WeightLoader(src, expected, "float32", "cpu").get("w")                 # the 32-bit run widens it exactly
    assert wide.dtype == torch.float32 and wide[0, 0].item() == 1.0009765625


def test_tied_head_is_optional_untied_head_is_required():
    tied = expected_tensors(Qwen3Config.from_dict(TINY_A).model_spec())
    assert tied["lm_head.weight"].optional
    tensors = {n: torch.zeros(s.shape) for n, s in tied.items() if n != "lm_head.weight"}
    check(DictSource(tensors), tied)
    untied = expected_tensors(Qwen3Config.from_dict(TINY_B).model_spec())
    with pytest.raises(WeightError, match="lm_head.weight"):
        check(DictSource({n: torch.zeros(s.shape) for n, s in untied.items() if n != "lm_head.weight"}), untied)


def test_storage_types():
    assert storage_dtype(torch.bfloat16, "bfloat16") == torch.bfloat16
    with pytest.raises(ValueError, match="rounding"):
        storage_dtype(torch.float16, "bfloat16")
    assert storage_dtype(torch.float16, "float32") == torch.float32
    assert storage_dtype(torch.float32, "bfloat16") == torch.float32   # a tensor stored in 32-bit stays so
    assert storage_dtype(torch.int64, "bfloat16") == torch.int32       # integer tables
    assert storage_dtype(torch.bfloat16, "float32") == torch.float32
    assert storage_dtype(torch.int16, "float32") == torch.int32
    with pytest.raises(ValueError):
        storage_dtype(torch.float32, "float16")
    expected = {"w": TensorSpec((2, 2)), "n": TensorSpec((2,), kind="norm"), "t": TensorSpec((3,), kind="table")}
    src = DictSource({"w": torch.ones(2, 2, dtype=torch.bfloat16), "n": torch.ones(2), "t": torch.arange(3)})
    load = WeightLoader(src, expected, "bfloat16", "cpu")
    assert (load.get("w").dtype, load.get("n").dtype, load.get("t").dtype) == (torch.bfloat16, torch.float32, torch.int32)
    load32 = WeightLoader(src, expected, "float32", "cpu")
    assert load32.get("w").dtype == torch.float32
    with pytest.raises(KeyError):
        load.get("other")
    assert load.get_concat(["w", "w"]).shape == (4, 2)


def test_random_weights_depend_only_on_seed_and_name(tmp_path):
    cfg = Qwen3Config.from_dict(TINY_A)
    expected = expected_tensors(cfg.model_spec())
    a, b, c = RandomSource(expected, 3), RandomSource(expected, 3), RandomSource(expected, 4)
    name = "model.layers.1.mlp.down_proj.weight"
    assert torch.equal(a.get(name), b.get(name)) and not torch.equal(a.get(name), c.get(name))
    only = RandomSource({name: expected[name]}, 3)
    assert torch.equal(only.get(name), a.get(name))     # independent of which other tensors exist
    w = a.get(name).float()
    assert abs(w.std().item() - expected[name].fan_in ** -0.5) < 0.02
    n = a.get("model.layers.0.input_layernorm.weight").float()
    assert n.min() >= 0.89 and n.max() <= 1.11 and n.std() > 0.01
    fixed = RandomSource(expected, 3, init=0.02).get(name).float()
    assert abs(fixed.std().item() - 0.02) < 0.002
    assert "lm_head.weight" not in a.names()            # tied: the head's tensor is not written

    folder = write_model_folder(cfg, str(tmp_path / "m"), seed=3)
    assert sorted(os.listdir(folder)) == ["config.json", "model.safetensors"]
    src = SafetensorsSource(folder)
    check(src, expected)
    assert torch.equal(src.get(name), a.get(name)) and src.info(name)[0] == torch.bfloat16
    again = Qwen3Config.load(folder)
    assert again == cfg


def test_duplicate_tensor_across_files_is_an_error(tmp_path):
    write_safetensors(str(tmp_path / "a.safetensors"), {"x": torch.zeros(2)})
    write_safetensors(str(tmp_path / "b.safetensors"), {"x": torch.zeros(2)})
    with pytest.raises(ValueError, match="held by both"):
        SafetensorsSource(str(tmp_path))
    with pytest.raises(FileNotFoundError):
        SafetensorsSource(str(tmp_path / "none") if os.makedirs(tmp_path / "none") is None else "")

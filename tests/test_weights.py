"""Weights: container checks, loading by name, one error for everything wrong, random
model folders (no GPU)."""
import json
import os
import struct

import pytest
import torch

from rbitnet_amd.config import LlamaConfig, load_config
from rbitnet_amd.engine.model import expected_tensors
from rbitnet_amd.errors import WeightError
from rbitnet_amd.weights import SafetensorsFile, WeightFolder, load_weights, save_file, write_random_model

from helpers import TINY_A, TINY_B


@pytest.fixture()
def folder(tmp_path):
    return write_random_model(str(tmp_path / "m"), TINY_A, seed=3)


def _rewrite(folder, change):
    path = os.path.join(folder, "model.safetensors")
    f = SafetensorsFile(path)
    tensors = {n: f.tensor(n).clone() for n in f.names()}
    change(tensors)
    save_file(path, list(tensors.items()))


def test_random_folder_loads_and_keeps_dtypes(folder):
    cfg, spec = load_config(folder)
    expected = expected_tensors(spec)
    got = load_weights(folder, expected, LlamaConfig.tensor_aliases)
    assert set(got) == set(expected)
    assert all(t.dtype == torch.bfloat16 for t in got.values())          # stored bf16 stays bf16
    assert got["model.embed_tokens.weight"].shape == (256, 64)
    # same seed, same values; another seed, other values; tensors do not depend on their order
    again = write_random_model(folder + "2", TINY_A, seed=3)
    other = write_random_model(folder + "3", TINY_A, seed=4)
    a = load_weights(again, expected)
    o = load_weights(other, expected)
    assert all(torch.equal(got[n], a[n]) for n in got)
    assert not torch.equal(got["lm_head.weight"], o["lm_head.weight"])
    gains = got["model.norm.weight"].float()
    assert abs(float(gains.mean()) - 1.0) < 0.02 and 0.005 < float(gains.std()) < 0.04
    mats = got["model.layers.1.mlp.up_proj.weight"].float()
    assert abs(float(mats.mean())) < 0.002 and 0.017 < float(mats.std()) < 0.023


def test_float32_storage_stays_float32(tmp_path):
    folder = write_random_model(str(tmp_path / "f"), TINY_A, seed=0, dtype=torch.float32)
    got = load_weights(folder, expected_tensors(load_config(folder)[1]))
    assert all(t.dtype == torch.float32 for t in got.values())


def test_one_error_lists_missing_unexpected_and_wrong_shapes(folder):
    def change(t):
        del t["model.layers.1.mlp.up_proj.weight"]
        del t["model.norm.weight"]
        t["model.layers.0.extra.weight"] = torch.zeros(3)
        t["model.layers.0.self_attn.k_proj.weight"] = torch.zeros(64, 64, dtype=torch.bfloat16)
    _rewrite(folder, change)
    with pytest.raises(WeightError) as e:
        load_weights(folder, expected_tensors(load_config(folder)[1]), LlamaConfig.tensor_aliases)
    msg = str(e.value)
    assert "missing tensors (2)" in msg and "model.layers.1.mlp.up_proj.weight" in msg and "model.norm.weight" in msg
    assert "unexpected tensors (1)" in msg and "model.layers.0.extra.weight" in msg
    assert "wrong shapes (1)" in msg and "expected [32, 64], found [64, 64]" in msg


def test_gguf_style_names_are_alternates(folder):
    def change(t):
        t["token_embd.weight"] = t.pop("model.embed_tokens.weight")
        t["blk.0.attn_q.weight"] = t.pop("model.layers.0.self_attn.q_proj.weight")
        t["blk.1.attn_output.weight"] = t.pop("model.layers.1.self_attn.o_proj.weight")
        t["output.weight"] = t.pop("lm_head.weight")
        t["output_norm.weight"] = t.pop("model.norm.weight")
    _rewrite(folder, change)
    got = load_weights(folder, expected_tensors(load_config(folder)[1]), LlamaConfig.tensor_aliases)
    assert "model.layers.0.self_attn.q_proj.weight" in got and "lm_head.weight" in got


def test_tied_model_has_no_head_and_ignores_one(tmp_path):
    folder = write_random_model(str(tmp_path / "b"), TINY_B, seed=1)
    spec = load_config(folder)[1]
    expected = expected_tensors(spec)
    assert "lm_head.weight" not in expected
    _rewrite(folder, lambda t: t.update({"lm_head.weight": torch.zeros(384, 96, dtype=torch.bfloat16)}))
    with pytest.raises(WeightError, match="unexpected"):
        load_weights(folder, expected)
    load_weights(folder, expected, ignored=["lm_head.weight"])


def test_container_is_checked(tmp_path):
    p = str(tmp_path / "x.safetensors")
    with open(p, "wb") as f:
        f.write(b"\x01\x02")
    with pytest.raises(WeightError, match="too short"):
        SafetensorsFile(p)
    with open(p, "wb") as f:
        f.write(struct.pack("<Q", 1 << 40) + b"{}")
    with pytest.raises(WeightError, match="header length"):
        SafetensorsFile(p)
    with open(p, "wb") as f:
        f.write(struct.pack("<Q", 4) + b"nope")
    with pytest.raises(WeightError, match="not valid JSON"):
        SafetensorsFile(p)

    def write(header, payload=b"\0" * 16):
        blob = json.dumps(header).encode()
        with open(p, "wb") as f:
            f.write(struct.pack("<Q", len(blob)) + blob + payload)

    write({"a": {"dtype": "F32", "shape": [2, 2], "data_offsets": [0, 32]}})
    with pytest.raises(WeightError, match="outside the file"):
        SafetensorsFile(p)
    write({"a": {"dtype": "F32", "shape": [2, 2], "data_offsets": [0, 8]}})
    with pytest.raises(WeightError, match="needs 16"):
        SafetensorsFile(p)
    write({"a": {"dtype": "F8_E4M3", "shape": [16], "data_offsets": [0, 16]}})
    with pytest.raises(WeightError, match="unsupported element type F8_E4M3"):
        SafetensorsFile(p)
    write({"a": {"dtype": "F32", "shape": [2], "data_offsets": [0, 8]},
           "b": {"dtype": "F32", "shape": [2], "data_offsets": [4, 12]}})
    with pytest.raises(WeightError, match="overlap"):
        SafetensorsFile(p)
    with pytest.raises(WeightError, match="no model.safetensors"):
        WeightFolder(str(tmp_path / "nothing"))


def test_sharded_folder(tmp_path, folder):
    f = SafetensorsFile(os.path.join(folder, "model.safetensors"))
    names = f.names()
    out = tmp_path / "sharded"
    out.mkdir()
    half = len(names) // 2
    save_file(str(out / "s1.safetensors"), [(n, f.tensor(n)) for n in names[:half]])
    save_file(str(out / "s2.safetensors"), [(n, f.tensor(n)) for n in names[half:]])
    index = {"weight_map": {n: ("s1.safetensors" if i < half else "s2.safetensors") for i, n in enumerate(names)}}
    (out / "model.safetensors.index.json").write_text(json.dumps(index))
    (out / "config.json").write_text(json.dumps(TINY_A))
    got = load_weights(str(out), expected_tensors(load_config(str(out))[1]))
    assert all(torch.equal(got[n], f.tensor(n)) for n in names)


def test_integer_tables_become_int32(tmp_path):
    from rbitnet_amd.parts.base import TensorSpec
    p = tmp_path / "t"
    p.mkdir()
    save_file(str(p / "model.safetensors"), [("idx", torch.arange(5, dtype=torch.int64)), ("w", torch.ones(2, 2))])
    got = load_weights(str(p), {"idx": TensorSpec((5,), role="table"), "w": TensorSpec((2, 2))})
    assert got["idx"].dtype == torch.int32 and got["w"].dtype == torch.float32
    with pytest.raises(WeightError, match="expected integers"):
        load_weights(str(p), {"w": TensorSpec((2, 2), role="table"), "idx": TensorSpec((5,), role="table")})

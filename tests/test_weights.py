"""Weights: reading by name, kept dtypes, the one error that lists everything, random models."""
import json
import os

import numpy as np
import pytest
import torch
from safetensors.torch import load_file, save_file

import helpers
from bare_cuda_4gib_amd.config import load_config
from bare_cuda_4gib_amd.engine import Model
from bare_cuda_4gib_amd.errors import WeightError
from bare_cuda_4gib_amd.weights import SafetensorsFile, load_weights, write_random_model


def _expected(folder):
    arch, cfg = load_config(folder)
    return Model(arch.describe(cfg)).expected_weights()


def test_random_model_folder_is_reproducible_and_readable_by_the_library(tmp_path):
    a = write_random_model(helpers.TINY_A, 0, str(tmp_path / "a"), "bfloat16")
    b = write_random_model(helpers.TINY_A, 0, str(tmp_path / "b"), "bfloat16")
    c = write_random_model(helpers.TINY_A, 1, str(tmp_path / "c"), "float32")
    ta, tb, tc = (load_file(os.path.join(d, "model.safetensors")) for d in (a, b, c))
    assert set(ta) == set(_expected(a)) and len(ta) == 3 + 2 * 9
    for name in ta:
        assert torch.equal(ta[name], tb[name]) and ta[name].dtype == torch.bfloat16
        assert tc[name].dtype == torch.float32
    assert torch.equal(ta["model.layers.1.input_layernorm.weight"], torch.ones(64, dtype=torch.bfloat16))
    w = tc["model.layers.0.mlp.up_proj.weight"]
    assert tuple(w.shape) == (176, 64) and abs(float(w.std()) - 0.02) < 2e-3 and abs(float(w.mean())) < 2e-3
    assert not torch.equal(ta["lm_head.weight"].float(), tc["lm_head.weight"])
    cfg = json.load(open(os.path.join(a, "config.json")))
    assert cfg["architectures"] == ["LlamaForCausalLM"] and cfg["hidden_size"] == 64
    # tied: no lm_head.weight is written
    t = load_file(os.path.join(write_random_model(helpers.TINY_B, 2, str(tmp_path / "t"), "float32"), "model.safetensors"))
    assert "lm_head.weight" not in t


def test_kept_dtypes(tmp_path):
    folder = write_random_model(helpers.TINY_A, 0, str(tmp_path / "m"), "bfloat16")
    path = os.path.join(folder, "model.safetensors")
    tensors = load_file(path)
    tensors["model.norm.weight"] = tensors["model.norm.weight"].float() * 1.001          # stored in 32-bit
    tensors["model.layers.0.mlp.up_proj.weight"] = tensors["model.layers.0.mlp.up_proj.weight"].half()
    save_file(tensors, path)
    w = load_weights(folder, _expected(folder))
    assert w["model.norm.weight"].dtype == torch.float32                                 # stays 32-bit
    assert torch.equal(w["model.norm.weight"], tensors["model.norm.weight"])
    assert w["lm_head.weight"].dtype == torch.bfloat16                                   # stays bfloat16
    assert torch.equal(w["lm_head.weight"], tensors["lm_head.weight"])
    half = w["model.layers.0.mlp.up_proj.weight"]
    assert half.dtype == torch.float16 and torch.equal(half, tensors["model.layers.0.mlp.up_proj.weight"])
    # on the device: a float16 tensor is kept in bfloat16 by the 16-bit path, widened by the 32-bit one
    from bare_cuda_4gib_amd.engine.runtime import Runtime
    cpu = torch.device("cpu")
    placed = Runtime(cpu, torch.bfloat16).place_weight(half)
    assert placed.dtype == torch.bfloat16 and torch.equal(placed, half.float().to(torch.bfloat16))
    assert torch.equal(Runtime(cpu, torch.float32).place_weight(half), half.float())
    assert Runtime(cpu, torch.bfloat16).place_weight(w["model.norm.weight"]).dtype == torch.float32


def test_integer_tables_become_int32(tmp_path):
    save_file({"t": torch.tensor([[1, 2], [3, 40000]], dtype=torch.int64)}, str(tmp_path / "x.safetensors"))
    f = SafetensorsFile(str(tmp_path / "x.safetensors"))
    assert f.tensor("t").dtype == torch.int32 and f.tensor("t").tolist() == [[1, 2], [3, 40000]]


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path, capsys):
    folder = write_random_model(helpers.TINY_A, 0, str(tmp_path / "m"), "float32")
    path = os.path.join(folder, "model.safetensors")
    good = load_file(path)
    tensors = dict(good)
    del tensors["model.layers.1.self_attn.k_proj.weight"]
    del tensors["model.norm.weight"]
    tensors["model.layers.0.mlp.down_proj.weight"] = torch.zeros(64, 175)
    tensors["model.layers.7.extra.weight"] = torch.zeros(3)
    tensors["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)            # tolerated buffer
    save_file(tensors, path)
    ignored = load_config(folder)[0].ignored_tensors
    assert ignored                                                # the architecture names what its checkpoints may carry
    with pytest.raises(WeightError) as e:
        load_weights(folder, _expected(folder), ignore=ignored)
    msg = str(e.value)
    assert "model.layers.1.self_attn.k_proj.weight" in msg and "model.norm.weight" in msg and "missing tensors (2)" in msg
    assert "model.layers.7.extra.weight" in msg and "unexpected tensors (1)" in msg
    assert "model.layers.0.mlp.down_proj.weight" in msg and "[64, 175]" in msg and "[64, 176]" in msg
    assert "inv_freq" not in msg


def test_unexpected_tensors_alone_are_a_warning(tmp_path, capsys):
    """A folder that holds everything the configuration needs, and more, loads: the tensors nobody
    asks for are listed once on standard error (the reference only looks up the names it needs,
    engine/src/loader.cpp:137-148); what the architecture says its checkpoints carry is not even listed."""
    folder = write_random_model(helpers.TINY_A, 0, str(tmp_path / "m"), "float32")
    path = os.path.join(folder, "model.safetensors")
    tensors = load_file(path)
    tensors["model.layers.7.extra.weight"] = torch.zeros(3)
    tensors["optimizer.step"] = torch.zeros(1)
    tensors["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)
    save_file(tensors, path)
    capsys.readouterr()
    w = load_weights(folder, _expected(folder), ignore=load_config(folder)[0].ignored_tensors)
    err = capsys.readouterr().err
    assert set(w) == set(_expected(folder)) and "model.layers.7.extra.weight" not in w
    assert err.count("warning") == 1 and "model.layers.7.extra.weight" in err and "optimizer.step" in err
    assert "inv_freq" not in err and "2 tensors" in err


def test_malformed_header_entries_name_the_tensor(tmp_path):
    p = tmp_path / "model.safetensors"
    for entry, word in (({"dtype": "F32", "data_offsets": [0, 16]}, "shape"),
                        ({"dtype": "F32", "shape": [4], "data_offsets": [0]}, "data_offsets"),
                        ({"dtype": "F32", "shape": [-4], "data_offsets": [0, 16]}, "shape"),
                        ({"dtype": "F32", "shape": [4], "data_offsets": [16, 0]}, "data_offsets"),
                        ("nonsense", "object")):
        header = json.dumps({"bad.tensor": entry}).encode()
        p.write_bytes(len(header).to_bytes(8, "little") + header + b"\0" * 16)
        with pytest.raises(WeightError) as e:
            SafetensorsFile(str(p))
        assert "bad.tensor" in str(e.value) and word in str(e.value)


def test_norm_spread_and_scaled_tensors(tmp_path):
    """The random-weights mode's two options: norm scales drawn around 1.0, a different draw for
    every norm, and tensors scaled by name."""
    a = load_file(os.path.join(write_random_model(helpers.TINY_A, 0, str(tmp_path / "a"), "float32", norm_std=0.1,
                                                  scales={"*.q_proj.weight": 8.0}), "model.safetensors"))
    plain = load_file(os.path.join(write_random_model(helpers.TINY_A, 0, str(tmp_path / "p"), "float32"), "model.safetensors"))
    n1, n2 = a["model.layers.0.input_layernorm.weight"], a["model.layers.0.post_attention_layernorm.weight"]
    assert not torch.equal(n1, n2) and abs(float(n1.mean()) - 1.0) < 0.05 and 0.05 < float(n1.std()) < 0.15
    assert not torch.equal(a["model.norm.weight"], a["model.layers.1.input_layernorm.weight"])
    assert abs(float(a["model.layers.0.self_attn.q_proj.weight"].std()) - 0.16) < 0.02
    assert abs(float(a["model.layers.0.self_attn.k_proj.weight"].std()) - 0.02) < 0.003
    assert torch.equal(plain["model.norm.weight"], torch.ones(64))


def test_file_errors(tmp_path):
    with pytest.raises(WeightError):
        load_weights(str(tmp_path), {})
    p = tmp_path / "model.safetensors"
    p.write_bytes(b"\x05\x00")
    with pytest.raises(WeightError) as e:
        SafetensorsFile(str(p))
    assert "truncated" in str(e.value)
    p.write_bytes((1000).to_bytes(8, "little") + b"{}")
    with pytest.raises(WeightError):
        SafetensorsFile(str(p))
    p.write_bytes((4).to_bytes(8, "little") + b"{{{{")
    with pytest.raises(WeightError):
        SafetensorsFile(str(p))
    header = json.dumps({"a": {"dtype": "F32", "shape": [4], "data_offsets": [0, 16]}}).encode()
    p.write_bytes(len(header).to_bytes(8, "little") + header + b"\0" * 8)               # data outside the file
    with pytest.raises(WeightError):
        SafetensorsFile(str(p))


def test_sharded_folder(tmp_path):
    folder = write_random_model(helpers.TINY_A, 0, str(tmp_path / "m"), "float32")
    tensors = load_file(os.path.join(folder, "model.safetensors"))
    names = sorted(tensors)
    half = len(names) // 2
    save_file({n: tensors[n] for n in names[:half]}, os.path.join(folder, "model-00001-of-00002.safetensors"))
    save_file({n: tensors[n] for n in names[half:]}, os.path.join(folder, "model-00002-of-00002.safetensors"))
    os.remove(os.path.join(folder, "model.safetensors"))
    wm = {n: ("model-00001-of-00002.safetensors" if i < half else "model-00002-of-00002.safetensors") for i, n in enumerate(names)}
    json.dump({"weight_map": wm}, open(os.path.join(folder, "model.safetensors.index.json"), "w"))
    w = load_weights(folder, _expected(folder))
    assert all(torch.equal(w[n], tensors[n]) for n in names)

"""Weights: the safetensors container, tensors by name, the one error that lists every mismatch,
dtypes that are kept, seeded random weights."""
import json
import os
import struct

import numpy as np
import pytest
import torch

from helpers import CONFIG_A, CONFIG_B, make_folder

import vipera_rs_amd  # noqa: F401
from vipera_rs_amd.config import config_from_dict
from vipera_rs_amd.errors import IoError, ParseError, UnsupportedError
from vipera_rs_amd.models import declare_model
from vipera_rs_amd.weights import (MATRIX, VECTOR, Checkpoint, SafetensorsFile, TensorSpec, WeightsError, kept_dtype,
                                   random_tensor, standard_normal, tensor_key, write_safetensors)


def test_written_files_are_read_back_by_the_safetensors_library(tmp_path):
    from safetensors.torch import load_file
    tensors = {"a": torch.arange(6, dtype=torch.float32).reshape(2, 3), "b": torch.ones(4, dtype=torch.bfloat16),
               "c": torch.tensor([1, -2, 3], dtype=torch.int32)}
    path = str(tmp_path / "x.safetensors")
    write_safetensors(path, tensors.items(), metadata={"format": "pt"})
    theirs = load_file(path)
    ours = SafetensorsFile(path)
    for name, tensor in tensors.items():
        assert torch.equal(theirs[name], tensor) and torch.equal(ours.read(name), tensor)
        assert ours.tensors[name].shape == tuple(tensor.shape)


def test_files_written_by_the_library_are_read(tmp_path):
    from safetensors.torch import save_file
    tensors = {"w": torch.randn(3, 5), "v": torch.randn(7).to(torch.bfloat16)}
    path = str(tmp_path / "lib.safetensors")
    save_file(tensors, path)
    ours = SafetensorsFile(path)
    assert torch.equal(ours.read("w"), tensors["w"]) and torch.equal(ours.read("v"), tensors["v"])


def _raw(tmp_path, header: dict, payload: bytes = b"", name="bad.safetensors", header_bytes=None):
    raw = header_bytes if header_bytes is not None else json.dumps(header).encode()
    path = str(tmp_path / name)
    with open(path, "wb") as handle:
        handle.write(struct.pack("<Q", len(raw)) + raw + payload)
    return path


def test_malformed_files_are_refused_with_the_tensor_named(tmp_path):
    with pytest.raises(ParseError, match="too short"):
        p = str(tmp_path / "tiny"); open(p, "wb").write(b"abc"); SafetensorsFile(p)
    with pytest.raises(ParseError, match="header length"):
        p = str(tmp_path / "long"); open(p, "wb").write(struct.pack("<Q", 1 << 40) + b"{}"); SafetensorsFile(p)
    with pytest.raises(ParseError, match="not valid JSON"):
        SafetensorsFile(_raw(tmp_path, {}, header_bytes=b"{oops"))
    with pytest.raises(ParseError, match="past the file"):
        SafetensorsFile(_raw(tmp_path, {"t": {"dtype": "F32", "shape": [4], "data_offsets": [0, 16]}}, b"\0" * 8))
    with pytest.raises(ParseError, match="needs 16 bytes"):
        SafetensorsFile(_raw(tmp_path, {"t": {"dtype": "F32", "shape": [4], "data_offsets": [0, 8]}}, b"\0" * 8))
    with pytest.raises(ParseError, match="overlap"):
        SafetensorsFile(_raw(tmp_path, {"a": {"dtype": "F32", "shape": [2], "data_offsets": [0, 8]},
                                        "b": {"dtype": "F32", "shape": [2], "data_offsets": [4, 12]}}, b"\0" * 12))
    with pytest.raises(UnsupportedError, match="F8_E4M3"):
        SafetensorsFile(_raw(tmp_path, {"t": {"dtype": "F8_E4M3", "shape": [1], "data_offsets": [0, 1]}}, b"\0"))
    with pytest.raises(ParseError, match="twice"):
        SafetensorsFile(_raw(tmp_path, {}, b"\0" * 8, header_bytes=(
            b'{"t":{"dtype":"F32","shape":[1],"data_offsets":[0,4]},"t":{"dtype":"F32","shape":[1],"data_offsets":[4,8]}}')))
    with pytest.raises(IoError):
        Checkpoint(str(tmp_path / "nothing_here"))


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    cfg = config_from_dict(CONFIG_A)
    specs = declare_model(cfg)
    folder = make_folder(tmp_path / "m", CONFIG_A, 0)
    Checkpoint(folder).check(specs)  # a matching folder passes
    from safetensors.torch import load_file, save_file
    tensors = load_file(os.path.join(folder, "model.safetensors"))
    del tensors["model.layers.1.mlp.up_proj.weight"]
    del tensors["model.norm.weight"]
    tensors["model.embed_positions.weight"] = torch.zeros(256, 64)   # nobody asked for it
    tensors["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)
    tensors["model.layers.0.self_attn.k_proj.weight"] = torch.zeros(64, 64)
    tensors["model.layers.0.self_attn.q_proj.bias"] = torch.zeros(32)
    save_file(tensors, os.path.join(folder, "model.safetensors"))
    with pytest.raises(WeightsError) as err:
        Checkpoint(folder).check(specs)
    e = err.value
    assert sorted(e.missing) == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"]
    assert sorted(e.unexpected) == ["model.embed_positions.weight", "model.layers.0.self_attn.rotary_emb.inv_freq"]
    assert sorted(n for n, _, _ in e.wrong_shapes) == ["model.layers.0.self_attn.k_proj.weight",
                                                       "model.layers.0.self_attn.q_proj.bias"]
    text = str(e)
    for needle in ("missing tensors (2)", "unexpected tensors (2)", "wrong shapes (2)", "[64, 64], expected [32, 64]"):
        assert needle in text


def test_sharded_folders_and_duplicates(tmp_path):
    from safetensors.torch import save_file
    folder = tmp_path / "sharded"
    folder.mkdir()
    save_file({"a": torch.ones(2)}, str(folder / "model-00001-of-00002.safetensors"))
    save_file({"b": torch.zeros(3)}, str(folder / "model-00002-of-00002.safetensors"))
    (folder / "model.safetensors.index.json").write_text(json.dumps(
        {"weight_map": {"a": "model-00001-of-00002.safetensors", "b": "model-00002-of-00002.safetensors"}}))
    ck = Checkpoint(str(folder))
    assert sorted(ck.names()) == ["a", "b"] and torch.equal(ck.read("b"), torch.zeros(3))
    save_file({"a": torch.ones(2)}, str(folder / "model-00002-of-00002.safetensors"))
    with pytest.raises(ParseError, match="appears in both"):
        Checkpoint(str(folder))


def test_what_dtype_a_tensor_keeps():
    m, v = TensorSpec("m", (2, 2), MATRIX), TensorSpec("v", (2,), VECTOR)
    bf, f32 = torch.bfloat16, torch.float32
    assert kept_dtype(m, bf, bf) == bf            # bfloat16 stays bfloat16
    assert kept_dtype(m, f32, bf) == bf           # a matrix takes the run's dtype whatever the file stores ...
    assert kept_dtype(m, torch.float16, bf) == bf
    assert kept_dtype(m, f32, bf, keep_float32=True) == f32   # ... unless 32-bit storage is asked to be kept
    assert kept_dtype(m, torch.float16, bf, keep_float32=True) == bf
    assert kept_dtype(m, bf, f32) == f32          # the 32-bit run widens everything
    assert kept_dtype(v, f32, bf) == f32          # a vector stored in 32-bit stays so
    assert kept_dtype(v, bf, bf) == f32           # norm weights and biases are always 32-bit
    assert kept_dtype(TensorSpec("t", (2,), "int_table"), torch.int64, bf) == torch.int32


def test_random_weights_are_seeded_per_tensor_and_well_distributed(tmp_path):
    spec = TensorSpec("model.layers.0.mlp.up_proj.weight", (128, 64), MATRIX)
    a = random_tensor(spec, 3, torch.float32)
    assert torch.equal(a, random_tensor(spec, 3, torch.float32))          # same seed, same values
    assert not torch.equal(a, random_tensor(spec, 4, torch.float32))      # another seed
    other = TensorSpec("model.layers.1.mlp.up_proj.weight", (128, 64), MATRIX)
    assert not torch.equal(a, random_tensor(other, 3, torch.float32))     # another name, another stream
    assert tensor_key(3, spec.name) != tensor_key(3, other.name)
    n = standard_normal(tensor_key(1, "x"), 200_000)
    assert abs(n.mean()) < 0.01 and abs(n.std() - 1.0) < 0.01 and abs(np.mean(n ** 3)) < 0.03
    assert abs(float(a.std()) - 0.02) < 0.002
    norm = random_tensor(TensorSpec("model.norm.weight", (4096,), VECTOR, "one_plus_normal"), 0, torch.float32)
    assert abs(float(norm.mean()) - 1.0) < 0.002 and abs(float(norm.std()) - 0.02) < 0.002
    # the order of generation does not matter: a folder's tensor equals the tensor made alone
    folder = make_folder(tmp_path / "m", CONFIG_B, 1)
    ck = Checkpoint(folder)
    assert torch.equal(ck.read(spec.name), random_tensor(TensorSpec(spec.name, (200, 96), MATRIX), 1, torch.float32))
    assert ck.info("lm_head.weight").shape == (300, 96) and ck.info("model.layers.2.self_attn.o_proj.weight").dtype == "F32"


def test_a_bfloat16_folder(tmp_path):
    folder = make_folder(tmp_path / "m", CONFIG_A, 0, torch.bfloat16)
    ck = Checkpoint(folder)
    assert {ck.info(n).dtype for n in ck.names()} == {"BF16"}
    ck.check(declare_model(config_from_dict(CONFIG_A)))


def test_a_tied_model_may_hold_an_output_matrix(tmp_path):
    cfg = config_from_dict(CONFIG_A)                        # tied embeddings
    folder = make_folder(tmp_path / "m", CONFIG_A, 0)
    specs = declare_model(cfg)
    assert [s.name for s in specs if s.optional] == ["lm_head.weight"]
    ck = Checkpoint(folder)
    assert "lm_head.weight" not in ck.names()               # random weights do not write it
    ck.check(specs)
    tensors = {name: ck.read(name) for name in ck.names()}
    ck.close()
    tensors["lm_head.weight"] = tensors["model.embed_tokens.weight"].clone()
    write_safetensors(os.path.join(folder, "model.safetensors"), tensors.items())
    ck = Checkpoint(folder)
    ck.check(specs)                                         # present: tolerated
    ck.close()
    tensors["lm_head.weight"] = torch.zeros(3, 64)
    write_safetensors(os.path.join(folder, "model.safetensors"), tensors.items())
    with pytest.raises(WeightsError) as err:
        Checkpoint(folder).check(specs)                     # but it has to be the output matrix's shape
    assert err.value.wrong_shapes == [("lm_head.weight", (3, 64), (256, 64))] and not err.value.unexpected


def test_a_shard_index_may_only_name_files_of_its_folder(tmp_path):
    folder = make_folder(tmp_path / "m", CONFIG_A, 0)
    outside = tmp_path / "elsewhere.safetensors"
    os.rename(os.path.join(folder, "model.safetensors"), outside)
    index = os.path.join(folder, "model.safetensors.index.json")
    for name in ("../elsewhere.safetensors", str(outside), "sub/../../elsewhere.safetensors", 7):
        with open(index, "w") as handle:
            json.dump({"weight_map": {"model.norm.weight": name}}, handle)
        with pytest.raises(ParseError, match="does not name a file of this folder"):
            Checkpoint(folder)
    os.rename(outside, os.path.join(folder, "part-1.safetensors"))
    with open(index, "w") as handle:
        json.dump({"weight_map": {"model.norm.weight": "part-1.safetensors"}}, handle)
    assert "model.norm.weight" in Checkpoint(folder).names()

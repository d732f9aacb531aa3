"""Weight loading: names, dtypes, ties, and one error for everything that is wrong."""
import json
import os

import pytest
import torch
from safetensors.torch import load_file, save_file

from conftest import TINY_A, TINY_B
from transformers_neuronx_amd.opt.config import OPTConfig
from transformers_neuronx_amd.engine.model import DecoderModel, model_param_decls
from transformers_neuronx_amd.opt.spec import opt_spec
from transformers_neuronx_amd.weights import (Checkpoint, TensorDict, WeightsError, check, load_tensors,
                                              target_dtype, write_random_model)


def _decls(raw):
    return model_param_decls(opt_spec(OPTConfig.from_dict(raw)))


def test_declared_names_are_the_checkpoint_names():
    names = {d.name for d in _decls(TINY_A)}
    assert "model.decoder.embed_tokens.weight" in names and "lm_head.weight" in names
    assert "model.decoder.embed_positions.weight" in names and "model.decoder.final_layer_norm.bias" in names
    for part in ("self_attn.q_proj.weight", "self_attn.k_proj.bias", "self_attn.v_proj.weight",
                 "self_attn.out_proj.bias", "self_attn_layer_norm.weight", "fc1.weight", "fc2.bias",
                 "final_layer_norm.bias"):
        assert f"model.decoder.layers.1.{part}" in names
    assert not any("project_in" in n for n in names)
    shapes = {d.name: d.shape for d in _decls(TINY_A)}
    assert shapes["model.decoder.embed_positions.weight"] == (130, 64)      # two rows more than positions
    assert shapes["model.decoder.layers.0.fc1.weight"] == (256, 64)
    b = {d.name: d.shape for d in _decls(TINY_B)}
    assert b["model.decoder.project_in.weight"] == (96, 48) and b["model.decoder.project_out.weight"] == (48, 96)
    assert b["model.decoder.embed_tokens.weight"] == (1000, 48)
    assert not any(n.endswith(".bias") for n in b)                          # no biases, no affine norms
    assert not any("layer_norm" in n for n in b)


def test_random_model_round_trip(tmp_path):
    cfg = OPTConfig.from_dict(TINY_A)
    folder = write_random_model(cfg, str(tmp_path / "m"), seed=7, dtype="bfloat16")
    again = write_random_model(cfg, str(tmp_path / "n"), seed=7, dtype="bfloat16")
    a, b = load_file(folder + "/model.safetensors"), load_file(again + "/model.safetensors")
    assert a.keys() == b.keys() and all(torch.equal(a[k], b[k]) for k in a)
    other = load_file(write_random_model(cfg, str(tmp_path / "o"), seed=8, dtype="bfloat16") + "/model.safetensors")
    assert not torch.equal(a["model.decoder.layers.0.fc1.weight"], other["model.decoder.layers.0.fc1.weight"])
    assert "lm_head.weight" not in a                                        # tied: not written
    assert a["model.decoder.layers.0.fc1.weight"].dtype == torch.bfloat16
    assert a["model.decoder.layers.0.fc1.bias"].dtype == torch.float32
    assert abs(float(a["model.decoder.final_layer_norm.weight"].mean()) - 1.0) < 0.05
    tensors = load_tensors(_decls(TINY_A), Checkpoint(folder), torch.bfloat16, "cpu")
    assert tensors["lm_head.weight"] is tensors["model.decoder.embed_tokens.weight"]      # one buffer
    assert tensors["model.decoder.layers.0.fc1.weight"].dtype == torch.bfloat16
    assert tensors["model.decoder.layers.0.self_attn_layer_norm.weight"].dtype == torch.float32
    assert torch.equal(tensors["model.decoder.layers.1.fc2.weight"], a["model.decoder.layers.1.fc2.weight"])
    up = load_tensors(_decls(TINY_A), Checkpoint(folder), torch.float32, "cpu")
    assert all(t.dtype == torch.float32 for t in up.values())
    assert torch.equal(up["model.decoder.layers.1.fc2.weight"], a["model.decoder.layers.1.fc2.weight"].float())


def test_dtype_rule():
    bf, f32, f16 = torch.bfloat16, torch.float32, torch.float16
    assert target_dtype("matrix", f16, bf) == bf and target_dtype("matrix", bf, bf) == bf
    assert target_dtype("matrix", f32, bf) == f32            # a tensor stored in 32-bit stays so
    assert target_dtype("matrix", f32, bf, cast_float32=True) == bf      # unless its rounding is asked for
    assert target_dtype("vector", f32, bf, cast_float32=True) == f32
    assert target_dtype("vector", bf, bf) == f32 and target_dtype("table", f16, bf) == bf
    assert target_dtype("matrix", bf, f32) == f32 and target_dtype("index", torch.int64, bf) == torch.int32


def test_one_error_lists_everything(tmp_path):
    cfg = OPTConfig.from_dict(TINY_A)
    folder = write_random_model(cfg, str(tmp_path / "m"), seed=0, dtype="float32")
    t = load_file(folder + "/model.safetensors")
    del t["model.decoder.layers.0.fc1.bias"]
    del t["model.decoder.layers.1.self_attn.q_proj.weight"]
    t["model.decoder.layers.0.fc3.weight"] = torch.zeros(2, 2)
    t["model.decoder.layers.1.fc2.weight"] = torch.zeros(64, 255)
    t["model.decoder.layers.1.fc2.bias"] = torch.zeros(64, dtype=torch.int32)
    save_file(t, folder + "/model.safetensors")
    with pytest.raises(WeightsError) as err:
        check(_decls(TINY_A), Checkpoint(folder))
    e = err.value
    assert sorted(e.missing) == ["model.decoder.layers.0.fc1.bias", "model.decoder.layers.1.self_attn.q_proj.weight"]
    assert e.unexpected == ["model.decoder.layers.0.fc3.weight"]
    assert e.wrong_shape == [("model.decoder.layers.1.fc2.weight", (64, 255), (64, 256))]
    assert [n for n, _ in e.wrong_dtype] == ["model.decoder.layers.1.fc2.bias"]
    text = str(e)
    for word in ("fc1.bias", "q_proj.weight", "fc3.weight", "[64, 255]", "[64, 256]", "floating"):
        assert word in text


def test_base_model_names_and_untied_head(tmp_path):
    cfg = OPTConfig.from_dict(TINY_A)
    folder = write_random_model(cfg, str(tmp_path / "m"), seed=0, dtype="float32")
    t = load_file(folder + "/model.safetensors")
    stripped = {k[len("model."):] if k.startswith("model.") else k: v for k, v in t.items()}
    got = load_tensors(_decls(TINY_A), TensorDict(stripped), torch.float32, "cpu", base_prefix="model.")
    assert torch.equal(got["model.decoder.layers.0.fc1.weight"], t["model.decoder.layers.0.fc1.weight"])
    # the prefix a base model's checkpoint lacks is the architecture's to name, not the loader's
    assert opt_spec(cfg).base_model_prefix == "model."
    with pytest.raises(WeightsError, match="missing"):
        load_tensors(_decls(TINY_A), TensorDict(stripped), torch.float32, "cpu")
    # a copy of the tied head in the file is accepted when it says what the table says, and not read
    with_head = dict(t, **{"lm_head.weight": t["model.decoder.embed_tokens.weight"].clone()})
    got = load_tensors(_decls(TINY_A), TensorDict(with_head), torch.float32, "cpu")
    assert got["lm_head.weight"] is got["model.decoder.embed_tokens.weight"]
    # a head that differs from the table it is tied to belongs to another model: refused
    with pytest.raises(WeightsError, match="tied tensors differ: lm_head.weight") as err:
        load_tensors(_decls(TINY_A), TensorDict(dict(t, **{"lm_head.weight": torch.zeros(512, 64)})),
                     torch.float32, "cpu")
    assert err.value.tied_differ == [("lm_head.weight", "model.decoder.embed_tokens.weight")]
    # untied: the head is its own tensor and must be there
    untied = _decls(dict(TINY_A, tie_word_embeddings=False))
    with pytest.raises(WeightsError, match="lm_head.weight"):
        check(untied, TensorDict(t))
    head = torch.randn(512, 64)
    got = load_tensors(untied, TensorDict(dict(t, **{"lm_head.weight": head})), torch.float32, "cpu")
    assert torch.equal(got["lm_head.weight"], head)


def test_no_checkpoint_file(tmp_path):
    with pytest.raises(FileNotFoundError, match="model.safetensors"):
        Checkpoint(str(tmp_path))


def test_sharded_checkpoint(tmp_path):
    cfg = OPTConfig.from_dict(TINY_A)
    folder = write_random_model(cfg, str(tmp_path / "m"), seed=0, dtype="float32")
    t = load_file(folder + "/model.safetensors")
    os.remove(folder + "/model.safetensors")
    names = sorted(t)
    halves = {"a.safetensors": names[::2], "b.safetensors": names[1::2]}
    weight_map = {}
    for fname, keys in halves.items():
        save_file({k: t[k] for k in keys}, os.path.join(folder, fname))
        weight_map.update({k: fname for k in keys})
    json.dump({"weight_map": weight_map}, open(os.path.join(folder, "model.safetensors.index.json"), "w"))
    got = load_tensors(_decls(TINY_A), Checkpoint(folder), torch.float32, "cpu")
    assert all(torch.equal(got[k], t[k]) for k in t)


def test_what_is_said_about_dtypes_at_load(tmp_path, capsys):
    """A bfloat16 engine says so when it keeps 32-bit matrices as they are (their products then run on the
    float32 kernel), rounds them when asked to, and says when float16 storage loses bits."""
    cfg = OPTConfig.from_dict(TINY_A)
    folder = write_random_model(cfg, str(tmp_path / "m"), seed=0, dtype="float32")
    kept = load_tensors(_decls(TINY_A), Checkpoint(folder), torch.bfloat16, "cpu")
    assert kept["model.decoder.layers.0.fc1.weight"].dtype == torch.float32
    assert "stored in 32-bit and stay so" in capsys.readouterr().err
    cast = load_tensors(_decls(TINY_A), Checkpoint(folder), torch.bfloat16, "cpu", cast_float32=True)
    assert cast["model.decoder.layers.0.fc1.weight"].dtype == torch.bfloat16
    assert cast["model.decoder.layers.0.fc1.bias"].dtype == torch.float32
    assert capsys.readouterr().err == ""
    t = {k: (v.half() if v.dim() == 2 else v) for k, v in load_file(folder + "/model.safetensors").items()}
    load_tensors(_decls(TINY_A), TensorDict(t), torch.bfloat16, "cpu")
    assert "stored in float16 and are rounded to bfloat16" in capsys.readouterr().err


def test_final_norm_can_be_left_out():
    decls = {d.name for d in _decls(dict(TINY_A, _remove_final_layer_norm=True))}
    assert "model.decoder.final_layer_norm.weight" not in decls
    assert "model.decoder.layers.1.final_layer_norm.weight" in decls
    assert "model.decoder.final_layer_norm.weight" in {d.name for d in _decls(TINY_A)}

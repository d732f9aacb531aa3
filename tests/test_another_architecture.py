"""An architecture that the package does not know: defined in tests/toy_architecture.py with config.json keys, parts,
tensor names and a kernel of its own, registered by its import, and taken through everything a model folder
goes through: the random-weights writer, the registry, the loader and its error, the step function under every
way of cutting, the entry point, and bin/trace_run as a program of its own. No file of the package names it."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch
from safetensors.torch import load_file, save_file

import schedules
import toy_architecture as toy
from transformers_neuronx_amd.config import EngineConfig, read_config
from transformers_neuronx_amd.config.model_config import ConfigError
from transformers_neuronx_amd.engine import StepEntry
from transformers_neuronx_amd.engine.factory import runner_from_folder
from transformers_neuronx_amd.weights import WeightsError, write_random_model

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SIZES = {"one": toy.TOY_ONE, "two": toy.TOY_TWO}


def _folder(tmp_path, name, seed=4, dtype="float32"):
    cfg = toy.ToyTurnConfig.from_dict(SIZES[name])
    folder = write_random_model(cfg, str(tmp_path / f"toy_{name}_{dtype}"), seed, dtype=dtype)
    return folder, cfg, load_file(os.path.join(folder, "model.safetensors"))


def _requests(cfg, lengths, seed):
    g = torch.Generator().manual_seed(seed)
    return {f"r{i}": torch.randint(0, cfg.words, (n,), generator=g).tolist() for i, n in enumerate(lengths)}


def _step_through(runner, cfg, weights, requests, tol):
    expected = {rid: toy.plain_logits(cfg, weights, toks) for rid, toks in requests.items()}
    for steps, place in (schedules.whole(requests), schedules.head_then_singles(requests, tail=8),
                         schedules.portions(requests),
                         schedules.mixed(requests, max_tokens=192, page=16, seed=5, tail=8, max_live=3)):
        for rec in steps:
            logits = runner.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in rec["entries"]])
            for row in range(logits.shape[0]):
                rid, pos = place[(rec["step"], row)]
                want = expected[rid][pos]
                err = float((logits[row].float().cpu() - want).abs().max() / expected[rid].abs().max())
                assert err < tol, (rec["step"], rid, pos, err)
            for rid in rec["end"]:
                runner.finish(rid)
            runner.cache.check()
        assert not runner.cache.requests


def test_the_folder_names_its_architecture(tmp_path):
    folder, cfg, weights = _folder(tmp_path, "one")
    raw = json.load(open(os.path.join(folder, "config.json")))
    assert raw["architectures"] == ["ToyTurnLM"] and raw["model_type"] == "toy_turn" and raw["shared_heads"] == 1
    arch, read = read_config(folder)
    assert arch is toy.ARCHITECTURE and read == cfg
    assert weights["blocks.0.attn.wk.weight"].shape == (32, 96) and "out_norm.weight" in weights
    # the model type alone finds it too, and its own checks speak of its own keys
    arch2, _ = read_config(_rewritten(folder, tmp_path / "by_type", lambda r: r.pop("architectures")))
    assert arch2 is arch
    with pytest.raises(ConfigError, match="required key 'shared_heads'"):
        read_config(_rewritten(folder, tmp_path / "short", lambda r: r.pop("shared_heads")))
    with pytest.raises(ConfigError, match="head sizes in 16s"):
        read_config(_rewritten(folder, tmp_path / "odd", lambda r: r.update(width=90)))


def _rewritten(folder, to, change):
    raw = json.load(open(os.path.join(folder, "config.json")))
    change(raw)
    os.makedirs(to, exist_ok=True)
    with open(os.path.join(to, "config.json"), "w") as fp:
        json.dump(raw, fp)
    return str(to)


@pytest.mark.parametrize("name", ["one", "two"])
def test_steps_on_the_host(tmp_path, name):
    folder, cfg, weights = _folder(tmp_path, name)
    runner = runner_from_folder(folder, EngineConfig(dtype="float32", kernels="reference", device="cpu", page_size=16,
                                                     max_tokens=192, max_num_seqs=4))
    _step_through(runner, cfg, weights, _requests(cfg, [70, 33, 100], 8), 2e-5)


def test_the_loader_lists_its_tensors(tmp_path):
    folder, cfg, weights = _folder(tmp_path, "one")
    broken = dict(weights)
    del broken["blocks.1.attn.down.weight"]
    broken["blocks.1.attn.sideways.weight"] = torch.zeros(2, 2)
    broken["blocks.2.mlp.up.weight"] = torch.zeros(72, 95)
    save_file(broken, os.path.join(folder, "model.safetensors"))
    with pytest.raises(WeightsError) as e:
        runner_from_folder(folder, EngineConfig(dtype="float32", kernels="reference", device="cpu", max_tokens=64))
    text = str(e.value)
    assert "blocks.1.attn.down.weight" in text and "blocks.1.attn.sideways.weight" in text
    assert "blocks.2.mlp.up.weight" in text and "expected [72, 96]" in text


def _greedy(cfg, weights, prompt, new):
    toks = list(prompt)
    for _ in range(new):
        toks.append(int(toy.plain_logits(cfg, weights, toks)[-1].argmax()))
    return toks


def test_generation_through_the_entry_point_on_the_host(tmp_path):
    from transformers_neuronx_amd import NeuronAutoModelForCausalLM
    from transformers_neuronx_amd.causal_lm import CausalLMForSampling
    folder, cfg, weights = _folder(tmp_path, "two")
    model = NeuronAutoModelForCausalLM.from_pretrained(folder, batch_size=2, amp="f32", n_positions=64, page_size=16,
                                                       kernels="reference", device="cpu")
    assert type(model) is CausalLMForSampling          # no class of its own: the architecture-free one serves
    model.to_neuron()
    ids = torch.tensor([[5, 200, 17, 3], [9, 9, 100, 42]])
    out = model.sample(ids, sequence_length=14, top_k=1)
    for row in range(2):
        assert out[row].tolist() == _greedy(cfg, weights, ids[row].tolist(), 10)
    with pytest.raises(ValueError, match="cannot be larger than position embedding's context size"):
        NeuronAutoModelForCausalLM.from_pretrained(folder, n_positions=cfg.longest + 1, kernels="reference",
                                                   device="cpu")


def test_a_package_that_cannot_be_imported_is_named(monkeypatch, tmp_path):
    folder, _, _ = _folder(tmp_path, "one")
    monkeypatch.setenv("TNX_ARCHITECTURE_PACKAGES", "toy_architecture, no_such_package_anywhere")
    with pytest.raises(ConfigError, match="no_such_package_anywhere"):
        read_config(folder)


# ---------------------------------------------------------------- on the GPU

DEV = "cuda:0"


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,tol", [("float32", 2e-5), ("bfloat16", 3e-2)])
@pytest.mark.parametrize("name", ["one", "two"])
def test_steps_on_the_gpu(tmp_path, name, dtype, tol):
    folder, cfg, weights = _folder(tmp_path, name, dtype=dtype)
    runner = runner_from_folder(folder, EngineConfig(dtype=dtype, device=DEV, page_size=16, max_tokens=192,
                                                     max_num_seqs=4))
    _step_through(runner, cfg, weights, _requests(cfg, [70, 33, 100], 8), tol)


@pytest.mark.gpu
def test_trace_run_takes_it_from_the_environment(tmp_path):
    """The program knows nothing of the architecture but what the environment names."""
    folder, cfg, weights = _folder(tmp_path, "two")
    requests = _requests(cfg, [40, 70], 13)
    expected = {rid: toy.plain_logits(cfg, weights, toks) for rid, toks in requests.items()}
    steps, place = schedules.mixed(requests, max_tokens=192, seed=1)
    env = dict(os.environ, TNX_ARCHITECTURE_PACKAGES="toy_architecture",
               PYTHONPATH=os.pathsep.join([os.path.join(ROOT, "tests"), os.environ.get("PYTHONPATH", "")]))
    text = "\n".join(json.dumps(s) for s in steps) + "\n"
    for dtype, tol in (("float32", 2e-5), ("bfloat16", 3e-2)):
        out = tmp_path / f"cli_{dtype}"
        proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype,
                               "--out", str(out), "--max-tokens", "192"], input=text, text=True, capture_output=True,
                              timeout=110, env=env)
        assert proc.returncode == 0, proc.stderr
        assert proc.stdout.split() == [w for s in steps for w in ("done", str(s["step"]))]
        for (step, row), (rid, pos) in place.items():
            got = np.fromfile(os.path.join(out, f"{step}.f32"), dtype="<f4").reshape(-1, cfg.words)[row]
            err = float(np.abs(got - expected[rid][pos].numpy()).max()) / float(expected[rid].abs().max())
            assert err < tol, (dtype, step, rid, pos, err)
    # without the variable the folder is refused, with the known names in the message
    env.pop("TNX_ARCHITECTURE_PACKAGES")
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", "float32",
                           "--out", str(tmp_path / "none"), "--max-tokens", "192"], input=text, text=True,
                          capture_output=True, timeout=110, env=env)
    assert proc.returncode != 0 and "ToyTurnLM" in proc.stderr and "OPTForCausalLM" in proc.stderr


@pytest.mark.gpu
def test_generation_through_the_entry_point_on_the_gpu(tmp_path):
    from transformers_neuronx_amd import NeuronAutoModelForCausalLM
    folder, cfg, weights = _folder(tmp_path, "one")
    model = NeuronAutoModelForCausalLM.from_pretrained(folder, batch_size=2, amp="f32", n_positions=64, page_size=16)
    model.to_neuron()
    ids = torch.tensor([[5, 150, 17, 3], [9, 9, 100, 42]])
    out = model.sample(ids, sequence_length=14, top_k=1)
    for row in range(2):
        assert out[row].tolist() == _greedy(cfg, weights, ids[row].tolist(), 10)

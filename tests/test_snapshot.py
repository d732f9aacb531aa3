"""Snapshots of steps (`engine/snapshot.py`): what a step read and gave, written to a folder, and the step run
again alone from it: on the host with the torch rendition of the kernels, for OPT and for the toy model of
the tests with its windowed pages and its state; on the GPU under `-m gpu`."""
import json
import os

import pytest
import torch

import schedules
from transformers_neuronx_amd import EngineConfig
from transformers_neuronx_amd.engine import StepEntry
from transformers_neuronx_amd.engine.factory import runner_from_folder
from transformers_neuronx_amd.engine.snapshot import StepSnapshots, main, replay_snapshot
from safetensors.torch import load_file


def _requests(vocab, lengths, seed):
    g = torch.Generator().manual_seed(seed)
    return {f"r{i}": torch.randint(3, vocab, (n,), generator=g).tolist() for i, n in enumerate(lengths)}


def _run_mixed(runner, requests, folder, keep):
    """A mixed schedule over few pages with the steps `keep` written; returns the steps as they were run."""
    runner.snapshots = StepSnapshots(folder, keep)
    steps, _ = schedules.mixed(requests, max_tokens=192, page=16, seed=2, tail=8, max_live=3)
    for rec in steps:
        runner.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in rec["entries"]])
        for rid in rec["end"]:
            runner.finish(rid)
    runner.snapshots = None
    return steps


def _check_replays(make_runner, steps, folder, keep, exact=True):
    for n in keep:
        path = os.path.join(folder, f"iter{n}")
        record = json.load(open(os.path.join(path, "step.json")))
        ran = steps[n]["entries"]
        assert [e["tokens"] for e in record["entries"]] == [list(e["tokens"]) for e in ran]
        assert [e["want"] for e in record["entries"]] == [list(e["want"]) for e in ran]
        saved = load_file(os.path.join(path, "outputs.safetensors"))
        assert ("logits" in saved) == any(e["want"] for e in ran)
        assert any(k.startswith("tap.") for k in saved)
        fresh = make_runner()
        diffs = replay_snapshot(path, fresh)
        assert set(diffs) == set(saved)
        assert max(diffs.values()) == 0.0 if exact else max(diffs.values()) < 1e-5, diffs
        assert not fresh.cache.requests            # and its requests are gone again
        fresh.cache.check()
    assert sorted(os.listdir(folder)) == sorted(f"iter{n}" for n in keep)


def test_a_step_written_and_run_again_on_the_host(tiny_folders, tmp_path):
    folder, cfg, _ = tiny_folders["B"]
    ecfg = EngineConfig(dtype="float32", kernels="reference", device="cpu", page_size=16, max_tokens=192, max_num_seqs=4)
    make = lambda: runner_from_folder(folder, ecfg)
    requests = _requests(cfg["vocab_size"], [70, 33, 100, 9], 8)
    out = str(tmp_path / "snap")
    keep = [1, 4, 9]
    steps = _run_mixed(make(), requests, out, keep)
    assert any(len(steps[n]["entries"]) > 1 for n in keep)      # a portion of a prompt beside decoded tokens
    _check_replays(make, steps, out, keep)
    # the comparison can fail: with other weights the same step gives other logits
    from conftest import TINY_B
    from transformers_neuronx_amd.opt.config import OPTConfig
    from transformers_neuronx_amd.weights.random_init import write_random_model
    write_random_model(OPTConfig.from_dict(TINY_B), str(tmp_path / "other"), 99, dtype="float32")
    other = runner_from_folder(str(tmp_path / "other"), ecfg)
    assert max(replay_snapshot(os.path.join(out, "iter4"), other).values()) > 1e-3
    # and the program that does the same from a command line
    assert main(["--model", folder, "--snapshot", os.path.join(out, "iter4"), "--kernels", "reference", "--device", "cpu"]) == 0


def _toy_runner(ops_kind, dtype, device):
    import toy_parts
    from transformers_neuronx_amd.cache import CacheManager
    from transformers_neuronx_amd.engine import DecoderModel, ModelRunner
    from transformers_neuronx_amd.kernels import make_ops
    from transformers_neuronx_amd.weights import TensorDict, random_tensors
    spec = toy_parts.toy_spec()
    model = DecoderModel(spec)
    tensors = random_tensors(model.param_decls(), spec.init_std, 3, torch.float32)
    ops = make_ops(ops_kind, dtype, device)
    model.load(TensorDict(tensors), ops, dtype, device)
    return ModelRunner(model, CacheManager(model.cache_needs(), 16, 12, 4, dtype, device), ops)


def test_a_step_with_windowed_pages_and_state_run_again_on_the_host(tmp_path):
    """The toy model: a window whose pages have been given back, state of fixed size in slots."""
    make = lambda: _toy_runner("reference", torch.float32, "cpu")
    requests = _requests(300, [70, 33, 100], 8)
    out = str(tmp_path / "snap")
    keep = [2, 7, 12]
    steps = _run_mixed(make(), requests, out, keep)
    record = json.load(open(os.path.join(out, "iter12", "step.json")))
    assert set(record["groups"]) == {"full", "window24"}
    assert any(p < 0 for row in record["groups"]["window24"]["table"] for p in row[:-1])     # pages the window let go
    assert any(k.startswith("state.") for k in load_file(os.path.join(out, "iter12", "inputs.safetensors")))
    _check_replays(make, steps, out, keep)


def test_snapshots_named_by_the_environment(tiny_folders, tmp_path, monkeypatch):
    folder, cfg, _ = tiny_folders["A"]
    monkeypatch.setenv("TNX_SNAPSHOT_PATH", str(tmp_path / "env"))
    monkeypatch.setenv("TNX_SNAPSHOT_STEPS", "[1]")
    ecfg = EngineConfig(dtype="float32", kernels="reference", device="cpu", page_size=16, max_tokens=64, max_num_seqs=2)
    runner = runner_from_folder(folder, ecfg)
    assert runner.snapshots is not None and runner.snapshots.steps == {1}
    runner.step([StepEntry("a", [5, 6, 7], [2])])
    runner.step([StepEntry("a", [8], [0])])
    assert os.listdir(tmp_path / "env") == ["iter1"]
    monkeypatch.delenv("TNX_SNAPSHOT_PATH")
    assert runner_from_folder(folder, ecfg).snapshots is None


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_step_written_and_run_again_on_the_gpu(tiny_folders, tiny_folders_bf16, tmp_path, dtype):
    """The HIP kernels give the same bits for the same step, whichever pages it lies in."""
    folder, cfg, _ = (tiny_folders if dtype == "float32" else tiny_folders_bf16)["C"]
    ecfg = EngineConfig(dtype=dtype, page_size=16, max_tokens=192, max_num_seqs=4)
    make = lambda: runner_from_folder(folder, ecfg)
    requests = _requests(cfg["vocab_size"], [70, 33, 100, 9], 8)
    out = str(tmp_path / "snap")
    keep = [1, 4, 9, 15]
    steps = _run_mixed(make(), requests, out, keep)
    _check_replays(make, steps, out, keep)


@pytest.mark.gpu
def test_the_command_line_writes_snapshots(tiny_folders, tmp_path, monkeypatch, capsys):
    """`opt_demo run --snapshot` (generation_demo.py:269, :551-554) names the folder in the environment; every
    step of the generation lies there afterwards, run-ahead steps with their tokens named by slot among them,
    and each runs again to the same bits."""
    from transformers_neuronx_amd.opt import demo
    folder, cfg, _ = tiny_folders["A"]
    monkeypatch.chdir(tmp_path)
    monkeypatch.setenv("TNX_SNAPSHOT_STEPS", "[0, 3, 4]")
    monkeypatch.setenv("TNX_SNAPSHOT_PATH", "")          # (so that what the command line sets is gone after the test)
    assert demo.main(["--amp", "f32", "run", folder, "--batch_size", "2", "--n_positions", "24", "--prompt_len", "7"]
                     + ["--snapshot"]) in (0, None)
    monkeypatch.delenv("TNX_SNAPSHOT_PATH", raising=False)
    out = tmp_path / "tnx_snapshot_f32_b2"
    assert sorted(os.listdir(out)) == ["iter0", "iter3", "iter4"]
    record = json.load(open(out / "iter3" / "step.json"))
    assert [len(e["tokens"]) for e in record["entries"]] == [1, 1] and record["entries"][0]["cached"] >= 7
    ecfg = EngineConfig(dtype="float32", page_size=record["page_size"], max_tokens=256, max_num_seqs=4)
    for n in (0, 3, 4):
        diffs = replay_snapshot(str(out / f"iter{n}"), runner_from_folder(folder, ecfg))
        assert max(diffs.values()) == 0.0, (n, diffs)
    capsys.readouterr()
    assert main(["--model", folder, "--snapshot", str(out / "iter4")]) == 0
    assert "logits: 0.000e+00" in capsys.readouterr().out

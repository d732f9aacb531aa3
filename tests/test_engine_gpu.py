"""The engine against the plain implementation, under every way of cutting and batching."""
import io
import json
import os

import numpy as np
import pytest
import torch

import plain_opt
import schedules
from conftest import TINY_A

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

# max |difference| of logits allowed, as a fraction of the largest |logit| of the request
TOL = {"float32": 2e-5, "bfloat16": 2e-2}


def _requests(cfg, lengths, seed):
    g = torch.Generator().manual_seed(seed)
    return {f"r{i}": torch.randint(3, cfg["vocab_size"], (n,), generator=g).tolist() for i, n in enumerate(lengths)}


def _expected(weights, cfg, requests):
    return {rid: plain_opt.forward_logits(weights, cfg, toks) for rid, toks in requests.items()}


def _run(folder, dtype, steps, max_tokens, page_size, tmp_path, name):
    from transformers_neuronx_amd.engine.replay import make_replay_runner, replay
    runner = make_replay_runner(folder, dtype, max_tokens, page_size, DEV)
    out = str(tmp_path / name)
    log = io.StringIO()
    replay((json.dumps(s) for s in steps), runner, out, log)
    assert log.getvalue().split() == [w for s in steps for w in ("done", str(s["step"]))]
    runner.cache.check()
    assert not runner.cache.requests, "requests left live at the end of the trace"
    return out, runner


def _compare(out, place, expected, vocab, dtype):
    worst = 0.0
    by_step = {}
    for (step, row), (rid, pos) in place.items():
        by_step.setdefault(step, []).append((row, rid, pos))
    for step, rows in by_step.items():
        got = np.fromfile(os.path.join(out, f"{step}.f32"), dtype="<f4").reshape(-1, vocab)
        assert got.shape[0] == len(rows)
        for row, rid, pos in rows:
            want = expected[rid][pos].numpy()
            scale = float(expected[rid].abs().max())
            err = float(np.abs(got[row] - want).max()) / scale
            worst = max(worst, err)
            assert err <= TOL[dtype], f"step {step} request {rid} position {pos}: error {err:.3e} of the logit range"
            if dtype == "float32":
                assert int(got[row].argmax()) == int(want.argmax())
    return worst


CASES = [("A", [5, 17, 31, 100, 128]), ("B", [1, 9, 40, 77, 120, 256]), ("C", [3, 64, 65, 150, 192])]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,lengths", CASES)
@pytest.mark.parametrize("page_size", [16, 64, 48])     # 48: no power of two, the general kernels take it
def test_schedules_agree_with_plain(tiny_folders, tiny_folders_bf16, tmp_path, dtype, name, lengths, page_size):
    folder, cfg, weights = (tiny_folders if dtype == "float32" else tiny_folders_bf16)[name]
    requests = _requests(cfg, lengths, seed=len(lengths))
    expected = _expected(weights, cfg, requests)
    longest = -(-max(lengths) // 64) * 64
    for kind, (steps, place), max_tokens in [
        ("whole", schedules.whole(requests), longest),
        ("singles", schedules.head_then_singles(requests), longest),
        ("portions", schedules.portions(requests), longest),
        ("mixed", schedules.mixed(requests, max_tokens=longest + 128, seed=3), longest + 128),
        ("mixed2", schedules.mixed(requests, max_tokens=2 * longest + 64, seed=4), 2 * longest + 64),
    ]:
        out, _ = _run(folder, dtype, steps, max_tokens, page_size, tmp_path, f"{kind}")
        _compare(out, place, expected, cfg["vocab_size"], dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_steps_that_want_nothing(tiny_folders, tiny_folders_bf16, tmp_path, dtype, name):
    """Portions and decoded tokens whose logits nobody asks for: the steps run, leave their keys and values,
    write no file, and the one row wanted at each request's end is right."""
    folder, cfg, weights = (tiny_folders if dtype == "float32" else tiny_folders_bf16)[name]
    requests = _requests(cfg, [5, 40, 77, 120], seed=3)
    expected = _expected(weights, cfg, requests)
    for made in (schedules.portions(requests), schedules.mixed(requests, max_tokens=256, page=16, seed=4)):
        steps, place = schedules.only_last(made)
        assert len(place) == len(requests) and any(not any(e["want"] for e in s["entries"]) for s in steps)
        out, _ = _run(folder, dtype, steps, 256, 16, tmp_path, f"last_{len(steps)}")
        assert sorted(os.listdir(out)) == sorted(f"{step}.f32" for step, _ in place)
        _compare(out, place, expected, cfg["vocab_size"], dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(tiny_folders, tiny_folders_bf16, tmp_path, dtype):
    """A short prompt, then 240 tokens one by one, across many pages."""
    folder, cfg, weights = (tiny_folders if dtype == "float32" else tiny_folders_bf16)["B"]
    requests = _requests(cfg, [250], seed=9)
    expected = _expected(weights, cfg, requests)
    steps, place = schedules.head_then_singles(requests, tail=240)
    out, _ = _run(folder, dtype, steps, 256, 16, tmp_path, "long")
    _compare(out, place, expected, cfg["vocab_size"], dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_first_tokens(tiny_folders, tiny_folders_bf16, tmp_path, dtype, name):
    """Prompts of one and two tokens, then single tokens: the first positions of a sequence."""
    folder, cfg, weights = (tiny_folders if dtype == "float32" else tiny_folders_bf16)[name]
    requests = _requests(cfg, [6, 7], seed=1)
    expected = _expected(weights, cfg, requests)
    steps = []
    for rid, first in (("r0", 1), ("r1", 2)):
        toks = requests[rid]
        steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": toks[:first],
                                                       "want": list(range(first))}], "end": []})
        for t in toks[first:]:
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": [t], "want": [0]}], "end": []})
        steps[-1]["end"] = [rid]
    steps, place = schedules._finish(steps)
    out, _ = _run(folder, dtype, steps, 64, 16, tmp_path, "first")
    _compare(out, place, expected, cfg["vocab_size"], dtype)


def test_pages_are_used_again_without_leaking(tiny_folders, tmp_path):
    """One page pool of the smallest size, request after request: every request sees pages its
    predecessor wrote, and its logits do not change."""
    folder, cfg, weights = tiny_folders["A"]
    requests = _requests(cfg, [60, 64, 33, 64, 17], seed=21)
    expected = _expected(weights, cfg, requests)
    steps, place = schedules.portions(requests, sizes=(19, 2, 30, 64))
    out, runner = _run(folder, "float32", steps, 64, 16, tmp_path, "reuse")
    assert runner.cache.groups["full"].pool.num_pages == 4
    _compare(out, place, expected, cfg["vocab_size"], "float32")


@pytest.mark.parametrize("amp", ["f32", "bf16"])
def test_greedy_generation_through_the_entry_point(tiny_folders, amp, tmp_path):
    from safetensors.torch import load_file
    from transformers_neuronx_amd import OPTForSampling
    from transformers_neuronx_amd.opt.config import OPTConfig
    from transformers_neuronx_amd.kernels import hip
    from transformers_neuronx_amd.weights import write_random_model
    # with weights as narrow as A's the greedy path repeats one token; a third model has A's sizes and
    # weights ten times as wide, so that its tokens differ from one another
    wide = str(tmp_path / "wide")
    write_random_model(OPTConfig.from_dict(dict(TINY_A, init_std=0.2)), wide, 11, dtype="float32")
    cases = [tiny_folders["A"], tiny_folders["B"],
             (wide, json.load(open(os.path.join(wide, "config.json"))), load_file(os.path.join(wide, "model.safetensors")))]
    for case, (folder, cfg, weights) in enumerate(cases):
        model = OPTForSampling.from_pretrained(folder, batch_size=3, amp=amp, n_positions=64, page_size=16,
                                               num_pages=9, max_num_batched_tokens=24).load()
        ids = torch.randint(3, cfg["vocab_size"], (3, 11), generator=torch.Generator().manual_seed(2))
        out = model.sample(ids, sequence_length=40, top_k=1)
        assert out.shape == (3, 40)
        if amp == "f32":
            for b in range(3):
                assert out[b].tolist() == plain_opt.greedy(weights, cfg, ids[b].tolist(), 29)
                assert case != 2 or len(set(out[b, 11:].tolist())) > 8
        else:
            # bfloat16 may part from the float32 choice where two logits are close: every chosen token
            # must be within the rounding of the best one under the plain implementation
            for b in range(3):
                toks = out[b].tolist()
                logits = plain_opt.forward_logits(weights, cfg, toks[:-1])
                for pos in range(10, 39):
                    row = logits[pos]
                    assert float(row.max() - row[toks[pos + 1]]) <= 3e-2 * float(row.abs().max())
    assert set(hip.loaded_libraries()) >= {"elementwise", "gemm", "attention", "sampling"}


def test_save_notes_the_built_kernels(tiny_folders, tmp_path):
    """`save` is the reference's way to keep what was compiled (base.py:39-48); here that is the kernels."""
    from transformers_neuronx_amd import OPTForSampling
    model = OPTForSampling.from_pretrained(tiny_folders["A"][0], batch_size=1, amp="bf16", n_positions=32).load()
    model.save(str(tmp_path / "artifacts"))
    noted = json.load(open(tmp_path / "artifacts" / "kernels.json"))
    from transformers_neuronx_amd.kernels import build
    # every registered module, those that parts of the tests brought among them
    assert set(noted) == set(build.modules()) >= {"elementwise", "gemm", "attention", "sampling", "probe"}
    assert all(os.path.exists(p) for p in noted.values())
    again = OPTForSampling.from_pretrained(tiny_folders["A"][0], batch_size=1, amp="bf16", n_positions=32)
    again.load(str(tmp_path / "artifacts")).to_neuron()
    assert again.is_compiled() and again.sample(torch.tensor([[5, 6, 7]]), 6).shape == (1, 6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_toy_parts_on_the_gpu(dtype):
    """A mixer with state of its own, registered by the test, beside full, windowed and cache-sharing
    attention, in a run order that names layers twice."""
    from test_engine_cpu import run_toy_model
    run_toy_model("hip", dtype, DEV, 2e-5 if dtype == torch.float32 else 3e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_toy_routed_parts_on_the_gpu(dtype):
    """A routed feed-forward and another position encoding, defined in the tests, on the HIP backend."""
    from test_engine_cpu import run_toy_routed_model
    run_toy_routed_model("hip", dtype, DEV, 2e-5 if dtype == torch.float32 else 3e-2)


def test_a_norm_that_only_scales_folded_into_the_products():
    """A model of the tests whose norms only scale (no mean, no bias) and ask the backend to fold them into the
    products that read them: decode steps of few rows run norm and product in one launch, recorded, and the
    logits are the plain implementation's."""
    import toy_parts
    from transformers_neuronx_amd.cache import CacheManager
    from transformers_neuronx_amd.engine import DecoderModel, ModelRunner, StepEntry
    from transformers_neuronx_amd.kernels import make_ops
    from transformers_neuronx_amd.kernels.hip import DeferredNorm
    from transformers_neuronx_amd.weights import TensorDict, random_tensors
    kw = dict(width=128, heads=4, kv_heads=2)
    spec = toy_parts.toy_spec_rotating(inner=256, vocab=160, tables=True, latent_layer=False, fold=True, **kw)
    model = DecoderModel(spec)
    tensors = random_tensors(model.param_decls(), spec.init_std, 4, torch.bfloat16)
    ops = make_ops("hip", torch.bfloat16, DEV)
    model.load(TensorDict(tensors), ops, torch.bfloat16, DEV)
    block = model.layers[0].block
    assert block.fold_mixer_norm and block.fold_feed_forward_norm
    assert isinstance(model.layers[0].mixer_norm.deferred(torch.zeros(2, 128, device=DEV)), DeferredNorm)
    runner = ModelRunner(model, CacheManager(model.cache_needs(), 16, 24, 4, torch.bfloat16, DEV), ops, use_graphs=True)
    requests = _requests(dict(vocab_size=160), [60, 33, 90], 10)
    expected = {rid: toy_parts.toy_rotating_plain_logits(tensors, toks, latent_layer=False, **kw) for rid, toks in requests.items()}
    ids = list(requests)
    runner.step([StepEntry(rid, requests[rid][:20], []) for rid in ids])
    for pos in range(20, 33):
        logits = runner.step([StepEntry(rid, [requests[rid][pos]], [0]) for rid in ids]).float().cpu()
        for i, rid in enumerate(ids):
            want = expected[rid][pos]
            assert float((logits[i] - want).abs().max() / want.abs().max()) < 3e-2, (rid, pos)
    assert runner.graph_replays == 13


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_toy_rotating_parts_on_the_gpu(dtype):
    """Queries and keys turned by an encoding of the tests, and a norm whose HIP kernel lives under tests/
    and is registered, compiled and called without a change to the package."""
    from test_engine_cpu import run_toy_rotating_model
    from transformers_neuronx_amd.kernels import hip
    run_toy_rotating_model("hip", dtype, DEV, 2e-5 if dtype == torch.float32 else 3e-2)
    assert "toy_norm" in hip.loaded_libraries()
    # the same encoding as pairwise tables: turned inside the projection's launch (the fused product of few
    # rows, the scatter after a library product, the float32 path), and decode steps replayed from recordings
    runner = run_toy_rotating_model("hip", dtype, DEV, 2e-5 if dtype == torch.float32 else 3e-2, in_the_projection=True)
    assert runner.graph_replays > 10


def test_benchmark_report_and_kernel_times(tiny_folders_bf16, capsys):
    """`opt_demo run --benchmark --profile`: the reference's report (warm-up, timed generations, latency
    percentiles) and the time of every kernel of a prompt step and a decode step."""
    from transformers_neuronx_amd.opt import demo
    folder = tiny_folders_bf16["C"][0]
    assert demo.main(["--amp", "bf16", "run", folder, "--batch_size", "2", "--n_positions", "40", "--prompt_len", "9",
                      "--top_k", "1", "--benchmark", "--profile", "--page_size", "16"]) in (0, None)
    text = capsys.readouterr().out
    report = json.loads(next(line for line in text.splitlines() if line.startswith("{")))
    assert report["iterations"] == 5 and report["inferences"] == 10 and report["context_length"] == 9
    pct = report["sequence_latency_percentiles"]
    assert 0 < pct["sequence_latency_p0"] <= pct["sequence_latency_p50"] <= pct["sequence_latency_p100"]
    assert report["e2e_output_token_throughput"] > 0 and report["mean_output_token_latency"] > 0
    assert report["mean_context_encoding_latency"] > 0
    for kernel in ("tnx_layernorm", "tnx_gemm_bf16", "tnx_attention_prefill", "tnx_attention_decode", "tnx_argmax"):
        assert kernel in text, kernel
    assert "prompt step" in text and "decode step" in text


def test_trace_run_as_a_program(tiny_folders, tmp_path):
    import subprocess
    import sys
    folder, cfg, weights = tiny_folders["A"]
    requests = _requests(cfg, [40, 70], seed=13)
    expected = _expected(weights, cfg, requests)
    steps, place = schedules.mixed(requests, max_tokens=192, seed=1)
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    for dtype in ("float32", "bfloat16"):
        out = tmp_path / f"cli_{dtype}"
        proc = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", folder,
                               "--dtype", dtype, "--out", str(out), "--max-tokens", "192"],
                              input="\n".join(json.dumps(s) for s in steps) + "\n", text=True,
                              capture_output=True, timeout=110)
        assert proc.returncode == 0, proc.stderr
        assert proc.stdout.split() == [w for s in steps for w in ("done", str(s["step"]))]
        _compare(str(out), place, expected, cfg["vocab_size"], dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16", "bfloat16 library"])
def test_recorded_decode_steps_equal_open_ones(tiny_folders, tiny_folders_bf16, dtype, monkeypatch):
    """Decode steps replayed from a recording give the logits of steps launched in the open, replay after
    replay, with prompt steps and other batch sizes in between. The third case sends every product of two rows
    and more to the vendor library, as batches of 17 and more do: its calls are recorded and replayed too."""
    from transformers_neuronx_amd.config import EngineConfig
    from transformers_neuronx_amd.engine import StepEntry
    from transformers_neuronx_amd.engine.factory import runner_from_folder
    from transformers_neuronx_amd.kernels.hip import HipOps
    if dtype.endswith("library"):
        dtype = "bfloat16"
        monkeypatch.setattr(HipOps, "library_rows", 2)
        monkeypatch.setattr(HipOps, "small_matrix", 0)
    folder, cfg, weights = (tiny_folders if dtype == "float32" else tiny_folders_bf16)["B"]
    requests = _requests(cfg, [60, 3, 90], seed=17)
    expected = _expected(weights, cfg, requests)

    def run(use_graphs):
        ecfg = EngineConfig(dtype=dtype, page_size=16, max_tokens=512, max_num_seqs=4, use_graphs=use_graphs)
        runner = runner_from_folder(folder, ecfg)
        rows = {}
        pos = {rid: 0 for rid in requests}

        def step(parts):
            entries = [StepEntry(rid, requests[rid][pos[rid]:pos[rid] + n], [n - 1]) for rid, n in parts]
            logits = runner.step(entries).clone()
            for i, (rid, n) in enumerate(parts):
                pos[rid] += n
                rows[(rid, pos[rid] - 1)] = logits[i].cpu()
        step([("r0", 20), ("r2", 50)])
        for _ in range(6):
            step([("r0", 1), ("r2", 1)])                 # recorded at batch 2
        step([("r1", 1)])                                 # a first token, batch 1
        for _ in range(2):
            step([("r0", 1), ("r1", 1), ("r2", 1)])      # batch 3
        step([("r0", 5), ("r2", 1)])                      # mixed: not recorded
        for _ in range(8):
            step([("r0", 1), ("r2", 1)])                 # batch 2 again: replayed
        return rows, runner.graph_replays

    open_rows, n_open = run(False)
    rec_rows, n_rec = run(True)
    assert n_open == 0 and n_rec == 6 + 1 + 2 + 8
    assert open_rows.keys() == rec_rows.keys()
    for key in open_rows:
        rid, p = key
        assert torch.equal(open_rows[key], rec_rows[key]), key
        want = expected[rid][p]
        assert float((rec_rows[key] - want).abs().max() / expected[rid].abs().max()) <= TOL[dtype]


LONG = dict(architectures=["OPTForCausalLM"], model_type="opt", vocab_size=300, hidden_size=128, num_hidden_layers=2,
            num_attention_heads=2, ffn_dim=256, max_position_embeddings=1100, init_std=0.08)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("batch,heads,total", [(2, 2, 1030), (9, 2, 1030), (8, 32, 530)])
def test_recorded_decoding_across_the_marks_of_256_keys(tmp_path, dtype, batch, heads, total):
    """Requests about as long as one another are decoded in blocks of 256 keys, and a recorded step is
    recorded again when the longest of them needs another block: from 250 to 1,030 tokens that happens four
    times. Every step is a recorded one; the logits at every mark (the three steps around it) and at every
    50th position are compared with the plain implementation, for the first and the last request. Nine requests
    of two heads are 18 (request, head) pairs, which the kernel cuts further than two requests; eight requests
    of 32 heads are a block for every compute unit as they are, stay whole, and are recorded once."""
    from safetensors.torch import load_file
    from transformers_neuronx_amd.config import EngineConfig
    from transformers_neuronx_amd.engine import StepEntry
    from transformers_neuronx_amd.engine.factory import runner_from_folder
    from transformers_neuronx_amd.opt.config import OPTConfig
    from transformers_neuronx_amd.weights import write_random_model
    folder = str(tmp_path / "long")
    raw = dict(LONG, num_attention_heads=heads, hidden_size=max(128, 16 * heads))
    write_random_model(OPTConfig.from_dict(raw), folder, seed=8, dtype=dtype)
    weights = {k: v.float() for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
    cfg = OPTConfig.from_dict(raw).to_dict()
    first = 250
    requests = _requests(cfg, [total - i % 3 for i in range(batch)], seed=batch)        # alike, not equal
    ids = list(requests)
    watched = [ids[0], ids[-1]]
    expected = {rid: plain_opt.forward_logits(weights, cfg, requests[rid]) for rid in watched}
    ecfg = EngineConfig(dtype=dtype, page_size=64, max_tokens=batch * 1088, max_num_seqs=batch, use_graphs=True)
    runner = runner_from_folder(folder, ecfg)
    runner.step([StepEntry(rid, requests[rid][:first], []) for rid in ids])
    looked = set(range(first, total - 3, 50)) | {m + d for m in (256, 512, 768, 1024) for d in (-2, -1, 0, 1)}
    worst = 0.0
    shapes = set()
    for pos in range(first, total - 3):
        logits = runner.step([StepEntry(rid, [requests[rid][pos]], [0]) for rid in ids])
        shapes.add(runner._last_ctx.plan_host["decode_shape"])
        if pos in looked:
            got = logits.float().cpu()
            for rid in watched:
                want = expected[rid][pos]
                err = float((got[ids.index(rid)] - want).abs().max() / expected[rid].abs().max())
                worst = max(worst, err)
                assert err <= TOL[dtype], (rid, pos, err)
                if dtype == "float32":
                    assert int(got[ids.index(rid)].argmax()) == int(want.argmax())
    assert runner.graph_replays == total - 3 - first
    marks = -(-(total - 3) // 256)
    assert shapes == {(k, True) for k in range(1, marks + 1)}
    # a recording for every launch that differs: the matrix-unit decode kernel's blocks a request (bfloat16)
    whole = dtype == "float32" or (batch, heads) == (8, 32)
    assert len(runner._recorded) == (1 if whole else marks)
    print(f"{dtype}, {batch} requests: worst error {worst:.2e} of the logit range")


def test_schedules_with_library_products(tiny_folders_bf16, tmp_path, monkeypatch):
    """The path long prompts take (vendor library for the plain products, our kernels around them), forced
    on the tiny model by lowering the row count it starts at."""
    from transformers_neuronx_amd.kernels.hip import HipOps
    monkeypatch.setattr(HipOps, "library_rows", 8)
    folder, cfg, weights = tiny_folders_bf16["A"]
    requests = _requests(cfg, [17, 100, 128], seed=5)
    expected = _expected(weights, cfg, requests)
    for kind, (steps, place) in (("whole", schedules.whole(requests)), ("portions", schedules.portions(requests)),
                                 ("mixed", schedules.mixed(requests, max_tokens=256, seed=6))):
        out, _ = _run(folder, "bfloat16", steps, 256, 16, tmp_path, f"lib_{kind}")
        _compare(out, place, expected, cfg["vocab_size"], "bfloat16")


FULL_SIZES = {
    # the layer sizes of four members of the family (reference: the 175B key set, gen_random_pretrained.py:105-140)
    "6.7b": dict(vocab_size=50272, hidden_size=4096, num_hidden_layers=2, num_attention_heads=32, ffn_dim=16384,
                 max_position_embeddings=2048, init_std=0.02),
    # heads of 80: no power of two
    "2.7b": dict(vocab_size=50272, hidden_size=2560, num_hidden_layers=2, num_attention_heads=32, ffn_dim=10240,
                 max_position_embeddings=2048, init_std=0.02),
    # 40 heads; 80 and 320 blocks of 64 columns, which the products share out otherwise than 64 and 256
    "13b": dict(vocab_size=50272, hidden_size=5120, num_hidden_layers=2, num_attention_heads=40, ffn_dim=20480,
                max_position_embeddings=2048, init_std=0.02),
    # the norm after each half, an embedding narrower than the model
    "350m": dict(vocab_size=50272, hidden_size=1024, num_hidden_layers=3, num_attention_heads=16, ffn_dim=4096,
                 max_position_embeddings=2048, word_embed_proj_dim=512, do_layer_norm_before=False, init_std=0.02),
}


@pytest.mark.parametrize("size", list(FULL_SIZES))
def test_full_layer_sizes_against_plain(size):
    """A few layers of the sizes of OPT-6.7B (width 4096, 32 heads of 128, inner width 16384, vocabulary
    50272), OPT-2.7B, OPT-13B and OPT-350m on bfloat16-stored random weights: the float32 engine and the bfloat16
    engine against the plain implementation, under a schedule that takes a long prompt in portions, decodes
    beside another prompt, and ends with recorded decode steps. The reference's own yardstick for a
    low-precision run against a float32 one is `allclose(atol=1.0, rtol=1e-3)` with equal argmax
    (generation_demo.py:437-443); here the bounds are those of the other tests."""
    from transformers_neuronx_amd.config import EngineConfig
    from transformers_neuronx_amd.opt.config import OPTConfig
    from transformers_neuronx_amd.engine import DecoderModel, StepEntry
    from transformers_neuronx_amd.engine.factory import build_runner
    from transformers_neuronx_amd.opt.spec import opt_spec
    from transformers_neuronx_amd.weights import TensorDict, random_tensors
    cfg = OPTConfig.from_dict(FULL_SIZES[size])
    raw = cfg.to_dict()
    spec = opt_spec(cfg)
    tensors = random_tensors(DecoderModel(spec).param_decls(), spec.init_std, 3, torch.bfloat16, DEV)
    g = torch.Generator().manual_seed(0)
    long = torch.randint(3, cfg.vocab_size, (420,), generator=g).tolist()
    short = torch.randint(3, cfg.vocab_size, (40,), generator=g).tolist()
    # (request, first token, count, wanted places) step by step
    plan = [[("a", 0, 300, [299])], [("a", 300, 110, [0, 109])], [("a", 410, 1, [0]), ("b", 0, 30, [29])]]
    plan += [[("a", 411 + i, 1, [0]), ("b", 30 + i, 1, [0])] for i in range(9)]
    toks = {"a": long, "b": short}
    # decode batches of every class of row counts: 40 requests (the products of 33 to 128 rows), 20 (the norm's
    # own kernel in front of the folded copies), 9 and 8 (the norm inside the product)
    crowd = [f"c{i}" for i in range(40)]
    for i, rid in enumerate(crowd):
        toks[rid] = torch.randint(3, cfg.vocab_size, (4 + i % 3 + 4,), generator=g).tolist()
    plan.append([(rid, 0, len(toks[rid]) - 4, [len(toks[rid]) - 5]) for rid in crowd])
    for k, live in enumerate((40, 20, 9, 8)):
        plan.append([(rid, len(toks[rid]) - 4 + k, 1, [0]) for rid in crowd[:live]])
    recorded = sum(all(n == 1 and w == [0] for _, _, n, w in step) for step in plan)
    # the plain implementation: each request whole, then the head on the wanted positions only
    weights = {k: v.float().cpu() for k, v in tensors.items()}
    hidden = {}
    for rid, t in toks.items():
        x = plain_opt.embed(torch.tensor(t), weights, raw)
        for i in range(cfg.num_hidden_layers):
            x = plain_opt.block(x, weights, raw, i)
        hidden[rid] = x
    places = [(rid, first + w) for step in plan for rid, first, n, want in step for w in want]
    want = torch.cat([plain_opt.head(hidden[rid][pos:pos + 1], weights, raw) for rid, pos in places])
    scale = float(want.abs().max())
    top2 = want.topk(2, dim=-1).values

    def run(dtype):
        ecfg = EngineConfig(dtype=dtype, page_size=64, max_tokens=1024 + 64 * len(crowd), max_num_seqs=2 + len(crowd))
        runner = build_runner(cfg, TensorDict(tensors), ecfg)
        rows = []
        for step in plan:
            rows.append(runner.step([StepEntry(rid, toks[rid][first:first + n], w) for rid, first, n, w in step])
                        .float().cpu())
        assert runner.graph_replays == recorded == 13
        return torch.cat(rows)

    for dtype in ("float32", "bfloat16"):
        got = run(dtype)
        err = float((got - want).abs().max()) / scale
        assert err <= TOL[dtype], (dtype, err)
        # where the plain implementation has a clear winner the engine names the same token
        clear = (top2[:, 0] - top2[:, 1]) > 4 * TOL[dtype] * scale
        assert bool(clear.any()), "no row has a clear winner: the comparison of choices would be empty"
        assert bool((got.argmax(-1) == want.argmax(-1))[clear].all())


def test_full_depth_bfloat16_against_float32():
    """All 32 layers of OPT-6.7B's sizes on the same random weights (drawn in bfloat16): the float32 engine and
    the bfloat16 engine generate from a 300-token prompt through `LLMEngine`, one step over the prompt and
    20 decode steps (recorded ones, with running ahead), the bfloat16 engine held to the float32 engine's
    tokens. The yardstick is the reference's own for a low-precision run against a float32 one
    (generation_demo.py:437-443: allclose(atol=1.0, rtol=1e-3) and the same token, step by step) with the
    plain distance beside it: a bfloat16 kernel that loses part of a sum over the depth shows here, where a
    two-layer model hides it. The float32 engine at this size holds 26.6 GB of weights."""
    from transformers_neuronx_amd.config import EngineConfig
    from transformers_neuronx_amd.engine.engine import LLMEngine
    from transformers_neuronx_amd.engine.factory import runner_from_random
    from transformers_neuronx_amd.opt.config import OPTConfig
    from transformers_neuronx_amd.testing import compare_precisions
    cfg = OPTConfig.from_dict(dict(FULL_SIZES["6.7b"], num_hidden_layers=32))
    prompt = torch.randint(3, cfg.vocab_size, (300,), generator=torch.Generator().manual_seed(11)).tolist()
    engines = []
    for dtype in (torch.float32, torch.bfloat16):
        ecfg = EngineConfig(dtype=dtype, page_size=64, max_tokens=384, max_num_seqs=1)
        engines.append(LLMEngine(runner_from_random(cfg, 5, ecfg, storage=torch.bfloat16), ecfg))
    report = compare_precisions(engines[0], engines[1], prompt, 21)
    print("full depth, bfloat16 against float32:", report)
    assert engines[1].runner.graph_replays >= 19
    assert report["rows"] == report["allclose_rows"] == 21, report
    assert report["rel"] <= TOL["bfloat16"], report
    assert report["clear_rows"] >= 5, report          # the comparison of choices is not empty
    assert report["clear_same"] == report["clear_rows"], report


def _odd(v, heads, hs, layers, ffn, proj, pre, act, bias, affine, eps):
    return dict(architectures=["OPTForCausalLM"], model_type="opt", vocab_size=v, hidden_size=heads * hs,
                num_hidden_layers=layers, num_attention_heads=heads, ffn_dim=ffn, max_position_embeddings=200,
                word_embed_proj_dim=proj or heads * hs, do_layer_norm_before=pre, activation_function=act,
                enable_bias=bias, layer_norm_elementwise_affine=affine, layer_norm_eps=eps, init_std=0.05)


# Sizes at the edges of what the kernels take: every head size class (16 .. 256, also ones only the general
# attention kernel takes), one head and many, widths and vocabularies that are no multiple of 8, 16 or 128,
# a feed-forward narrower than a tile, an embedding narrower than the model.
ODD = [
    _odd(257, 1, 16, 1, 24, None, True, "relu", True, True, 1e-5),
    _odd(1001, 5, 48, 2, 200, 56, True, "gelu", True, True, 1e-5),
    _odd(50, 7, 80, 1, 72, None, False, "relu", False, True, 1e-4),
    _odd(333, 3, 112, 2, 328, 40, True, "gelu_new", True, False, 1e-5),
    _odd(1234, 2, 144, 1, 520, None, True, "relu", True, True, 1e-5),
    _odd(777, 1, 256, 1, 264, 24, False, "gelu", True, True, 1e-5),
    _odd(130, 9, 32, 2, 8, None, True, "relu", True, True, 1e-5),
    _odd(4099, 6, 64, 1, 1000, None, True, "relu", True, True, 1e-5),
    _odd(96, 2, 128, 1, 136, None, True, "relu", True, True, 1e-5),
    _odd(513, 11, 16, 3, 176, 8, True, "relu", False, False, 1e-3),
    # inner sizes of products that are no multiple of 8 (bfloat16 rows are read 16 bytes at a time; such
    # matrices are filled up when they are loaded) and embedding rows of an odd number of elements
    _odd(211, 2, 32, 2, 37, 33, True, "gelu", True, True, 1e-5),
    _odd(97, 3, 16, 1, 1, 1, False, "relu", False, False, 1e-4),
    _odd(300, 4, 64, 2, 1001, 127, True, "relu", True, True, 1e-5),
]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("index", range(len(ODD)))
def test_odd_sizes(tmp_path, dtype, index):
    from safetensors.torch import load_file
    from transformers_neuronx_amd.opt.config import OPTConfig
    from transformers_neuronx_amd.weights import write_random_model
    raw = ODD[index]
    folder = str(tmp_path / "model")
    write_random_model(OPTConfig.from_dict(raw), folder, index, dtype=dtype)
    weights = load_file(os.path.join(folder, "model.safetensors"))
    requests = _requests(raw, [3, 70, 129, 200], seed=index)
    expected = _expected(weights, raw, requests)
    for kind, (steps, place), max_tokens, page_size in [
        ("singles", schedules.head_then_singles(requests), 256, 16),
        ("mixed", schedules.mixed(requests, max_tokens=384, seed=index), 384, 64),
    ]:
        out, _ = _run(folder, dtype, steps, max_tokens, page_size, tmp_path, kind)
        _compare(out, place, expected, raw["vocab_size"], dtype)


def test_command_line_dump_and_analyze(tiny_folders, tmp_path, capsys):
    """`opt_demo run --dump_logits` writes the logits each token was chosen from; `analyze` compares two
    runs by the reference's yardstick (generation_demo.py:404-443) and fails when they differ."""
    from transformers_neuronx_amd.opt.config import OPTConfig
    from transformers_neuronx_amd.opt import demo
    folder, cfg, weights = tiny_folders["A"]
    prompt = [5, 17, 3, 200, 9]
    dirs = {}
    for amp in ("bf16", "f32"):
        dirs[amp] = str(tmp_path / f"logits_{amp}")
        demo.main(["--amp", amp, "run", folder, "--batch_size", "2", "--n_positions", "24", "--prompt_ids",
                   ",".join(map(str, prompt)), "--top_k", "1", "--dump_logits", dirs[amp],
                   "--dump_logits_limit", "-1"])
    steps = sorted(os.listdir(dirs["f32"]), key=lambda f: int(f[:-3]))
    assert len(steps) == 24 - len(prompt)
    # the dumped float32 logits are the plain implementation's, token by token, along the greedy path
    # (top_k 1; the reference's loop never picks the end-of-sequence token, sampling.py:143-144)
    eos = OPTConfig.from_dict(cfg).eos_token_id
    seq = list(prompt)
    for i, name in enumerate(steps):
        got = torch.load(os.path.join(dirs["f32"], name), weights_only=True)
        assert got.shape == (2, cfg["vocab_size"])
        ref = plain_opt.forward_logits(weights, cfg, seq)[-1]
        torch.testing.assert_close(got[0], ref, rtol=1e-4, atol=1e-4)
        torch.testing.assert_close(got[1], ref, rtol=1e-4, atol=1e-4)
        ref = ref.clone()
        ref[eos] = float("-inf")
        seq.append(int(ref.argmax()))
    assert demo.main(["analyze", "-d", dirs["bf16"], dirs["f32"]]) == 0
    # a spoiled dump is found
    bad = str(tmp_path / "bad")
    os.makedirs(bad)
    for name in steps:
        t = torch.load(os.path.join(dirs["f32"], name), weights_only=True)
        if name == "3.pt":
            t = t.clone()
            t[0, int(t[0].argmin())] = 1e3
        torch.save(t, os.path.join(bad, name))
    assert demo.main(["analyze", "-d", bad, dirs["f32"]]) == 1
    assert "step 3" in capsys.readouterr().out


def _drawn_case(seed):
    """A configuration, a precision, a page size, requests and a way of cutting them, all drawn from `seed`."""
    rng = np.random.default_rng(seed)
    hs = int(rng.choice([16, 32, 48, 64, 64, 64, 80, 96, 128, 128, 128, 160, 256]))
    heads = max(1, min(int(rng.integers(1, 7)), 768 // hs))
    hidden = heads * hs
    raw = dict(architectures=["OPTForCausalLM"], model_type="opt", vocab_size=int(rng.integers(40, 1500)),
               hidden_size=hidden, num_hidden_layers=int(rng.integers(1, 4)), num_attention_heads=heads,
               ffn_dim=int(rng.choice([8, 72, 128, 200, 256, 384, 520, 1024])),
               max_position_embeddings=int(rng.choice([300, 700])),
               word_embed_proj_dim=int(rng.choice([hidden, hidden, 48, 136])),
               do_layer_norm_before=bool(rng.random() < 0.7),
               activation_function=str(rng.choice(["relu", "gelu", "gelu_new"])),
               enable_bias=bool(rng.random() < 0.7), layer_norm_elementwise_affine=bool(rng.random() < 0.7),
               layer_norm_eps=float(rng.choice([1e-5, 1e-3])), init_std=float(rng.choice([0.02, 0.03, 0.05])))
    dtype = "bfloat16" if rng.random() < 0.7 else "float32"
    page = int(rng.choice([16, 32, 48, 64, 64, 128]))
    most = raw["max_position_embeddings"] - 2
    lengths = [int(min(most, rng.choice([rng.integers(1, 40), rng.integers(40, 300), rng.integers(200, 698)])))
               for _ in range(int(rng.integers(2, 13)))]
    max_live = int(rng.integers(1, 13))
    tail = int(rng.choice([4, 16, 40]))
    requests = _requests(raw, lengths, seed)
    rounded = sorted((-(-n // page) * page for n in lengths), reverse=True)
    kind = str(rng.choice(["mixed", "mixed", "portions", "singles"]))
    if kind == "mixed":
        max_tokens = sum(rounded[:max(1, max_live // 2)]) + page
        steps, place = schedules.mixed(requests, max_tokens=max_tokens, page=page, seed=seed, tail=tail,
                                       max_live=max_live)
    else:
        max_tokens = rounded[0] + page
        steps, place = (schedules.portions(requests) if kind == "portions"
                        else schedules.head_then_singles(requests, tail=tail))
    return raw, dtype, page, requests, max_tokens, steps, place


@pytest.mark.parametrize("seed", range(100, 124))
def test_drawn_configurations_and_schedules(tmp_path, seed):
    """Sizes, options, precision, page size, up to twelve requests of up to 698 tokens, up to twelve of them
    live, and the way they are cut into steps: all drawn from the seed, against the plain implementation."""
    from safetensors.torch import load_file
    from transformers_neuronx_amd.opt.config import OPTConfig
    from transformers_neuronx_amd.weights import write_random_model
    raw, dtype, page, requests, max_tokens, steps, place = _drawn_case(seed)
    folder = write_random_model(OPTConfig.from_dict(raw), str(tmp_path / "model"), seed, dtype=dtype)
    weights = load_file(os.path.join(folder, "model.safetensors"))
    expected = _expected(weights, raw, requests)
    out, _ = _run(folder, dtype, steps, max_tokens, page, tmp_path, "drawn")
    _compare(out, place, expected, raw["vocab_size"], dtype)


def test_command_line_options_of_the_reference(tiny_folders, capsys):
    """`opt_demo run` with the options of the reference's demos that mean something on one GPU: rows of
    different lengths (`--various`), an end-of-sequence token of the caller's, the accepted no-ops; and
    `--quantize`, which is refused."""
    import re
    from transformers_neuronx_amd.opt import demo
    folder, cfg, weights = tiny_folders["A"]
    base = ["--amp", "f32", "run", folder, "--batch_size", "3", "--n_positions", "20", "--prompt_len", "6",
            "--top_k", "1", "--unroll", "4", "--context_length_estimate", "16", "--continuous_batching"]

    def generated(extra):
        demo.main(base + extra)
        text = capsys.readouterr().out
        rows = re.findall(r"\[([\d,\s]+)\]", text[text.index("generated_sequence="):])
        return [[int(t) for t in r.replace(",", " ").split()] for r in rows]
    rows = generated(["--various", "--simple_sample_eos_token_override", "-1"])
    assert len(rows) == 3 and all(len(r) == 20 for r in rows)
    pad = cfg.get("pad_token_id", 1)
    for b, row in enumerate(rows):
        start = (b * 2) % 6
        assert row[:start] == [pad] * start
        want = plain_opt.greedy(weights, cfg, row[start:6], 14)      # nothing banned, nothing stops it
        assert row[start:] == want, (b, row, want)
    # a token the first row is known to generate ends that row: what follows is that token again
    stop = rows[0][9]
    again = generated(["--various", "--simple_sample_eos_token_override", str(stop)])
    first = rows[0].index(stop, 6)
    assert again[0][:first + 1] == rows[0][:first + 1] and set(again[0][first:]) == {stop}
    with pytest.raises(SystemExit, match="quantize"):
        demo.main(base + ["--quantize"])


def test_weight_copies_within_a_number_of_bytes(tiny_folders_bf16, tmp_path):
    """A model whose tile-ordered copies do not all fit gets those a number of bytes allows, the matrices with
    the fewest rows first, and the LayerNorm is folded into those that got one: the logits are the same
    with none, with some and with all."""
    from transformers_neuronx_amd.config import EngineConfig
    from transformers_neuronx_amd.engine.factory import runner_from_folder
    from transformers_neuronx_amd.kernels.hip import PreparedWeight
    folder, cfg, weights = tiny_folders_bf16["C"]        # width 128, inner width 256: every matrix can have a copy
    requests = _requests(cfg, [40, 9], seed=2)
    expected = _expected(weights, cfg, requests)
    steps, place = schedules.head_then_singles(requests, tail=6)
    seen = {}
    for name, kw in (("none", dict(weight_copies=False)), ("all", dict(weight_copies=True)),
                     ("some", dict(weight_copy_bytes=224 << 10))):
        runner = runner_from_folder(folder, EngineConfig(dtype="bfloat16", page_size=16, max_tokens=128, max_num_seqs=4,
                                                         device=DEV, **kw))
        held = [w for layer in runner.model.layers for w in (layer.mixer.w_qkv, layer.mixer.w_out, layer.feed_forward.w1,
                                                             layer.feed_forward.w2)]
        assert all(isinstance(w, PreparedWeight) for w in held)
        seen[name] = [(tuple(w.tensor.shape), w.tiles is not None or w.folded is not None) for w in held]
        rows = {}
        for rec in steps:
            from transformers_neuronx_amd.engine import StepEntry
            logits = runner.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in rec["entries"]]).float().cpu()
            for row in range(logits.shape[0]):
                rid, pos = place[(rec["step"], row)]
                err = float((logits[row] - expected[rid][pos]).abs().max() / expected[rid].abs().max())
                assert err <= TOL["bfloat16"], (name, rec["step"], rid, pos, err)
            for rid in rec["end"]:
                runner.finish(rid)
    assert not any(c for _, c in seen["none"]) and all(c for _, c in seen["all"])
    # 224 KB: by rising rows, the output products (128 x 128, 32 KB each) and fc2 (128 x 256, 64 KB each) of both
    # layers; then no fc1 (256 x 128), QKV (384 x 128) or head fits what is left
    assert sorted(shape for shape, c in seen["some"] if c) == [(128, 128), (128, 128), (128, 256), (128, 256)]

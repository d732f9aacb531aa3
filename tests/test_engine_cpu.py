"""The engine's host logic (cache, batching, scheduler, sampler) with the plain torch rendition of the
kernels, on the CPU: the same comparisons the GPU tests make with the HIP kernels."""
import io
import json

import numpy as np
import pytest
import torch

import plain_opt
import schedules
from conftest import TINY
from transformers_neuronx_amd.config import EngineConfig
from transformers_neuronx_amd.opt.config import OPTConfig
from transformers_neuronx_amd.engine import StepEntry
from transformers_neuronx_amd.engine.engine import LLMEngine
from transformers_neuronx_amd.engine.scheduler import PENDING
from transformers_neuronx_amd.engine.factory import runner_from_folder
from transformers_neuronx_amd.sampling import SamplingParams


def _runner(folder, max_tokens, page_size=16, **kw):
    cfg = EngineConfig(dtype="float32", kernels="reference", device="cpu", page_size=page_size,
                       max_tokens=max_tokens, max_num_seqs=8, **kw)
    return runner_from_folder(folder, cfg), cfg


def _requests(vocab, lengths, seed):
    g = torch.Generator().manual_seed(seed)
    return {f"r{i}": torch.randint(3, vocab, (n,), generator=g).tolist() for i, n in enumerate(lengths)}


@pytest.mark.parametrize("name,lengths", [("A", [5, 17, 31, 100]), ("B", [1, 9, 40, 77, 120])])
def test_schedules_on_the_host(tiny_folders, tmp_path, name, lengths):
    from transformers_neuronx_amd.engine.replay import replay
    folder, cfg, weights = tiny_folders[name]
    requests = _requests(cfg["vocab_size"], lengths, 2)
    expected = {rid: plain_opt.forward_logits(weights, cfg, toks) for rid, toks in requests.items()}
    for kind, (steps, place), max_tokens in [
        ("whole", schedules.whole(requests), 128),
        ("singles", schedules.head_then_singles(requests), 128),
        ("portions", schedules.portions(requests), 128),
        ("mixed", schedules.mixed(requests, max_tokens=256, seed=1), 256),
    ]:
        runner, _ = _runner(folder, max_tokens)
        out = tmp_path / f"{name}_{kind}"
        replay((json.dumps(s) for s in steps), runner, str(out), io.StringIO())
        runner.cache.check()
        for (step, row), (rid, pos) in place.items():
            got = np.fromfile(out / f"{step}.f32", dtype="<f4").reshape(-1, cfg["vocab_size"])[row]
            assert np.abs(got - expected[rid][pos].numpy()).max() < 1e-5, (kind, step, rid, pos)


def test_step_refuses_what_it_cannot_run(tiny_folders):
    folder, cfg, _ = tiny_folders["A"]
    runner, _ = _runner(folder, 64)
    with pytest.raises(ValueError, match="vocabulary"):
        runner.step([StepEntry("a", [5, 512], [0])])
    with pytest.raises(ValueError, match="vocabulary"):
        runner.step([StepEntry("a", [5, -1], [0])])       # only the engine may name a token kept on the device
    with pytest.raises(ValueError, match="vocabulary"):
        LLMEngine(runner, EngineConfig(dtype="float32", kernels="reference", device="cpu")).add_request(
            [3, -2], SamplingParams(max_new_tokens=2))
    with pytest.raises(ValueError, match="twice"):
        runner.step([StepEntry("a", [5], [0]), StepEntry("a", [6], [0])])
    with pytest.raises(ValueError, match="outside"):
        runner.step([StepEntry("a", [5, 6], [2])])
    with pytest.raises(ValueError, match="positions"):
        runner.step([StepEntry("b", [5] * 129, [])])
    assert runner.step([StepEntry("c", [5, 6, 7], [])]) is None          # nothing wanted: it still runs
    assert runner.cache.num_tokens("c") == 3


@pytest.mark.parametrize("name", ["A", "B"])
def test_generation_does_not_depend_on_the_schedule(tiny_folders, name):
    """Greedy and sampled tokens are the same whether requests run alone, together, in small portions, or
    with so few pages that some are put back and computed again."""
    folder, cfg, weights = tiny_folders[name]
    prompts = list(_requests(cfg["vocab_size"], [1, 9, 40, 77], 3).values())
    params = [SamplingParams(max_new_tokens=12, do_sample=False, ignore_eos=True),
              SamplingParams(max_new_tokens=12, temperature=0.8, seed=11, ignore_eos=True),
              SamplingParams(max_new_tokens=12, temperature=1.2, top_k=20, top_p=0.9, seed=5, ignore_eos=True),
              SamplingParams(max_new_tokens=12, do_sample=False, ignore_eos=True)]

    def generate(max_tokens, budget, together):
        runner, ecfg = _runner(folder, max_tokens, max_num_batched_tokens=budget)
        engine = LLMEngine(runner, ecfg)
        if together:
            outs = engine.generate(prompts, params)
        else:
            outs = [engine.generate([p], [sp])[0] for p, sp in zip(prompts, params)]
        runner.cache.check()
        assert not runner.cache.requests
        return outs, engine.scheduler.num_preemptions

    alone, _ = generate(512, 512, together=False)
    assert alone[0] == plain_opt.greedy(weights, cfg, prompts[0], 12)[len(prompts[0]):]
    assert alone[3] == plain_opt.greedy(weights, cfg, prompts[3], 12)[len(prompts[3]):]
    together, n0 = generate(512, 512, together=True)
    portions, _ = generate(512, 24, together=True)
    tight, n = generate(160, 32, together=True)            # 10 pages of 16 for 175 tokens: some go back
    assert n0 == 0 and n > 0
    assert alone == together == portions == tight


@pytest.mark.parametrize("name", ["A", "B"])
def test_running_ahead_changes_nothing_but_the_call_that_reports(tiny_folders, name):
    """With `run_ahead` a step is started before the tokens of the step before it are read. Requests that
    stop at their end-of-sequence token (found out one step late), at their length, that arrive while
    others run, and that are put back for want of pages generate what they generate without it, and every
    token is reported once, in order, the last one of a request marked as such."""
    folder, cfg, weights = tiny_folders[name]
    prompts = list(_requests(cfg["vocab_size"], [3, 9, 40, 77, 20, 5], 8).values())
    free = [SamplingParams(max_new_tokens=14, do_sample=False, ignore_eos=True),
            SamplingParams(max_new_tokens=14, temperature=0.9, seed=4, ignore_eos=True)] * 3

    def generate(run_ahead, params, max_tokens=512, budget=64):
        runner, ecfg = _runner(folder, max_tokens, max_num_batched_tokens=budget, run_ahead=run_ahead)
        engine = LLMEngine(runner, ecfg)
        seen, ends = {}, {}
        ids = [engine.add_request(p, sp) for p, sp in zip(prompts[:4], params[:4])]
        calls = 0
        while engine.has_work:
            for out in engine.step():
                assert out.req_id not in ends, "a token after the last one"
                seen.setdefault(out.req_id, []).append(out.token)
                if out.finished:
                    ends[out.req_id] = out.finish_reason
            calls += 1
            if calls == 3:                     # two more arrive while the others run
                ids += [engine.add_request(p, sp) for p, sp in zip(prompts[4:], params[4:])]
        runner.cache.check()
        assert not runner.cache.requests
        outs = [engine.requests[i].output for i in ids]
        assert [seen[i] for i in ids] == outs and set(ends) == set(ids)
        assert all(t >= 0 for o in outs for t in o)
        return outs, [ends[i] for i in ids], engine.scheduler.num_preemptions

    plain, reasons, _ = generate(False, free)
    assert reasons == ["length"] * 6
    assert generate(True, free)[:2] == (plain, reasons)
    # each request now stops at the token it generated fifth, unless that token came earlier already
    stopping = [SamplingParams(max_new_tokens=14, do_sample=sp.do_sample, temperature=sp.temperature, seed=sp.seed,
                               eos_token_id=out[4]) for sp, out in zip(free, plain)]
    want = [out[:out.index(out[4]) + 1] for out in plain]
    for run_ahead in (False, True):
        outs, reasons, _ = generate(run_ahead, stopping)
        assert outs == want and reasons == ["eos"] * 6
    # and with so few pages that requests are put back and computed again
    late = [b if i == 3 else a for i, (a, b) in enumerate(zip(free, stopping))]
    want = [b if i == 3 else a for i, (a, b) in enumerate(zip(plain, want))]
    for run_ahead in (False, True):
        outs, reasons, n = generate(run_ahead, late, max_tokens=160, budget=32)
        assert outs == want and reasons == ["eos" if i == 3 else "length" for i in range(6)] and n > 0


@pytest.mark.parametrize("run_ahead", [False, True])
def test_prompts_first_ends_when_pages_run_out(tiny_folders, run_ahead):
    """With `prompts_first` decoding requests wait for prompts, but a prompt that was put back for want of
    pages can only go on when the decoding requests have gone on and ended: they must not wait for it. The
    same holds when more requests wait than there are slots. The tokens are those of the other order."""
    folder, cfg, weights = tiny_folders["A"]
    prompts = list(_requests(cfg["vocab_size"], [30, 30, 30, 30, 30], 6).values())
    sp = SamplingParams(max_new_tokens=40, do_sample=False, ignore_eos=True)

    def generate(prompts_first, max_tokens, max_num_seqs=8):
        cfg_ = EngineConfig(dtype="float32", kernels="reference", device="cpu", page_size=16, max_tokens=max_tokens,
                            max_num_seqs=max_num_seqs, prompts_first=prompts_first, run_ahead=run_ahead)
        runner = runner_from_folder(folder, cfg_)
        engine = LLMEngine(runner, cfg_)
        ids = [engine.add_request(p, sp) for p in prompts]
        for _ in range(2000):
            if not engine.has_work:
                break
            engine.step()
        assert not engine.has_work, "the engine makes no progress"
        runner.cache.check()
        return [engine.requests[i].output for i in ids], engine.scheduler.num_preemptions

    want, _ = generate(False, 512)
    tight, n = generate(True, 128)               # 8 pages of 16 for 5 x 69 tokens
    assert n > 0 and tight == want
    few_slots, _ = generate(True, 512, max_num_seqs=2)
    assert few_slots == want


def test_a_step_that_plans_nothing_while_work_waits_raises(tiny_folders):
    folder, cfg, _ = tiny_folders["A"]
    runner, ecfg = _runner(folder, 128)
    engine = LLMEngine(runner, ecfg)
    engine.add_request([5, 6, 7], SamplingParams(max_new_tokens=4))
    engine.scheduler.schedule = lambda: []          # a scheduler that has work and plans none of it
    with pytest.raises(RuntimeError, match="no progress"):
        engine.run()
    with pytest.raises(RuntimeError, match="no progress"):      # a caller's own loop over step() meets it too
        while engine.has_work:
            engine.step()
    # the entry point's loop: a pool that the scheduler cannot plan the batch into
    from transformers_neuronx_amd import OPTForSampling
    model = OPTForSampling.from_pretrained(folder, batch_size=1, amp="f32", n_positions=32, kernels="reference",
                                           device="cpu").load()
    model.engine.scheduler.schedule = lambda: []
    with pytest.raises(RuntimeError, match="no progress"):
        model.sample(torch.tensor([[5, 6, 7]]), 8)


def test_end_tokens_of_any_integer_type():
    import numpy as np
    assert SamplingParams(eos_token_id=np.int64(7)).eos_ids == (7,)
    assert SamplingParams(eos_token_id=torch.tensor(7)).eos_ids == (7,)
    assert SamplingParams(eos_token_id=[np.int32(7), 9]).eos_ids == (7, 9)
    assert SamplingParams(eos_token_id=None).eos_ids == ()
    for bad in (7.5, "seven", [7, 1.5]):
        with pytest.raises(ValueError, match="eos_token_id"):
            SamplingParams(eos_token_id=bad)


def test_sampled_tokens_follow_the_plain_sampler(tiny_folders):
    folder, cfg, weights = tiny_folders["A"]
    prompt = _requests(cfg["vocab_size"], [13], 4)["r0"]
    sp = SamplingParams(max_new_tokens=6, temperature=0.7, top_k=8, top_p=0.95, seed=99, ignore_eos=True)
    runner, ecfg = _runner(folder, 128)
    out = LLMEngine(runner, ecfg).generate([prompt], sp)[0]
    toks = list(prompt)
    for n in range(6):
        logits = plain_opt.forward_logits(weights, cfg, toks)[-1]
        tok = plain_opt.sample_row(logits, plain_opt.philox_uniform(99, n), top_k=8, top_p=0.95, temperature=0.7)
        assert out[n] == tok
        toks.append(tok)


def test_forward_by_sequence_ids(tiny_folders):
    """With `continuous_batching` in the NeuronConfig `forward` is driven the way the reference's serving
    integration drives it (base.py:575-637): prompts go in one at a time under their `seq_ids`, then the
    sequences decode together, in any order, and a sequence id is used again for a new prompt."""
    from transformers_neuronx_amd import OPTForSampling
    from transformers_neuronx_amd.config import ContinuousBatchingConfig, NeuronConfig
    folder, cfg, weights = tiny_folders["B"]
    nc = NeuronConfig(continuous_batching=ContinuousBatchingConfig(max_num_seqs=3, max_model_len=64), padding_side="right")
    model = OPTForSampling.from_pretrained(folder, batch_size=3, amp="f32", n_positions=64, neuron_config=nc,
                                           kernels="reference", device="cpu", page_size=16).load()
    a, b = _requests(cfg["vocab_size"], [11, 4], 12).values()

    def last(tokens):
        return plain_opt.forward_logits(weights, cfg, tokens)[-1]
    la = model(torch.tensor([a]), torch.arange(11).unsqueeze(0), torch.tensor([2]))
    lb = model(torch.tensor([b]), torch.arange(4).unsqueeze(0), torch.tensor([0]))
    torch.testing.assert_close(la[0], last(a), atol=1e-5, rtol=1e-5)
    torch.testing.assert_close(lb[0], last(b), atol=1e-5, rtol=1e-5)
    both = model(torch.tensor([[7], [9]]), torch.tensor([[4], [11]]), torch.tensor([0, 2]))      # b first, then a
    torch.testing.assert_close(both[0], last(b + [7]), atol=1e-5, rtol=1e-5)
    torch.testing.assert_close(both[1], last(a + [9]), atol=1e-5, rtol=1e-5)
    with pytest.raises(ValueError, match="holds"):
        model(torch.tensor([[5]]), torch.tensor([[9]]), torch.tensor([0]))
    again = model(torch.tensor([a[:6]]), torch.arange(6).unsqueeze(0), torch.tensor([0]))          # row 0 anew
    torch.testing.assert_close(again[0], last(a[:6]), atol=1e-5, rtol=1e-5)
    only_a = model(torch.tensor([[3]]), torch.tensor([[12]]), torch.tensor([2]))                   # row 2 went on
    torch.testing.assert_close(only_a[0], last(a + [9, 3]), atol=1e-5, rtol=1e-5)


def test_generation_config_options(tiny_folders):
    """`GenerationConfig` as the reference's on-device generation reads it (config.py:106-139): a value a
    batch line, a global top-k above the lines' own, a least number of tokens for top-p, and the constant
    0.5 in place of random numbers."""
    from transformers_neuronx_amd import OPTForSampling
    from transformers_neuronx_amd.config import GenerationConfig
    folder, cfg, weights = tiny_folders["A"]
    prompt = _requests(cfg["vocab_size"], [9], 6)["r0"]
    model = OPTForSampling.from_pretrained(folder, batch_size=3, amp="f32", n_positions=32, kernels="reference",
                                           device="cpu").load()
    gen = GenerationConfig(do_sample=True, top_k=[1, 30, 0], top_p=[1.0, 0.02, 0.5], temperature=[1.0, 0.9, 1.4],
                           top_p_min_tokens=[1, 5, 2], global_top_k=20, deterministic=True, per_batch_line=True,
                           dynamic=True)
    out = model.sample(torch.tensor([prompt] * 3), sequence_length=15, generation_config=gen)
    for b, (k, p, t, least) in enumerate([(1, 1.0, 1.0, 1), (20, 0.02, 0.9, 5), (20, 0.5, 1.4, 2)]):
        toks = list(prompt)
        for n in range(6):
            logits = plain_opt.forward_logits(weights, cfg, toks)[-1]
            tok = plain_opt.sample_row(logits, 0.5, top_k=k, top_p=p, temperature=t, min_tokens_to_keep=least)
            assert int(out[b, len(toks)]) == tok, (b, n)
            toks.append(tok)
    # the second line is not greedy: five tokens stay and 0.5 falls past the first of them
    assert out[1].tolist() != out[0].tolist()


def test_entry_point_in_the_reference_manner(tiny_folders, tmp_path):
    from transformers_neuronx_amd import OPTForSampling
    folder, cfg, weights = tiny_folders["A"]
    model = OPTForSampling.from_pretrained(folder, batch_size=2, amp="f32", n_positions=48, kernels="reference",
                                           device="cpu", page_size=16)
    with pytest.raises(RuntimeError, match="load"):
        model.sample(torch.tensor([[5, 6]]), 8)
    assert not model.is_compiled()
    model.load(str(tmp_path))            # the reference's folder of compiled artifacts: nothing to take from it
    model.to_neuron()
    assert model.is_compiled()
    ids = torch.tensor([[5, 9, 200, 31], [7, 7, 100, 3]])
    out = model.sample(ids, sequence_length=12, top_k=1)
    assert out.shape == (2, 12) and torch.equal(out[:, :4], ids)
    for b in range(2):
        assert out[b].tolist() == plain_opt.greedy(weights, cfg, ids[b].tolist(), 8)
    sampled = model.sample(ids, sequence_length=12, top_k=50)
    assert sampled.shape == (2, 12) and not (sampled == cfg.get("eos_token_id", 2))[:, 4:].any()
    # forward in the reference's form: prompt pass, then one token at the next cache id
    logits = model(ids)
    want = torch.stack([plain_opt.forward_logits(weights, cfg, ids[b].tolist())[-1] for b in range(2)])
    torch.testing.assert_close(logits, want, atol=1e-5, rtol=1e-5)
    nxt = torch.tensor([[11], [12]])
    logits = model(nxt, torch.tensor([4]))
    want = torch.stack([plain_opt.forward_logits(weights, cfg, ids[b].tolist() + nxt[b].tolist())[-1]
                        for b in range(2)])
    torch.testing.assert_close(logits, want, atol=1e-5, rtol=1e-5)
    with pytest.raises(ValueError, match="cache_ids"):
        model(nxt, torch.tensor([9]))
    # rows padded on the left up to start_ids: the padding is dropped
    padded = torch.tensor([[1, 1, 5, 9], [7, 7, 100, 3]])
    logits = model(padded, None, torch.tensor([2, 0]))
    torch.testing.assert_close(logits[0], plain_opt.forward_logits(weights, cfg, [5, 9])[-1], atol=1e-5, rtol=1e-5)
    # every position's logits (`output_all_logits`, config.py:91): `[batch, tokens, vocab]`, zeros under the padding
    model.neuron_config.output_all_logits = True
    logits = model(padded, None, torch.tensor([2, 0]))
    assert logits.shape == (2, 4, cfg["vocab_size"]) and not logits[0, :2].any()
    torch.testing.assert_close(logits[0, 2:], plain_opt.forward_logits(weights, cfg, [5, 9]), atol=1e-5, rtol=1e-5)
    torch.testing.assert_close(logits[1], plain_opt.forward_logits(weights, cfg, [7, 7, 100, 3]), atol=1e-5, rtol=1e-5)
    model.neuron_config.output_all_logits = False
    # a smaller batch after a larger one: the rows it does not name give back what they held
    model(ids)
    assert sorted(model.engine.runner.cache.requests) == [("row", 0), ("row", 1)]
    logits = model(ids[1:])
    assert sorted(model.engine.runner.cache.requests) == [("row", 0)]
    model.engine.runner.cache.check()
    torch.testing.assert_close(logits[0], plain_opt.forward_logits(weights, cfg, ids[1].tolist())[-1], atol=1e-5, rtol=1e-5)
    model.reset()
    assert not model.engine.runner.cache.requests
    # a streamer gets one token of every row at a time and is told the end (sampling.py:159-160, :172-173),
    # also when the rows' prompts differ in length and enter the cache in different steps
    class Collect:
        def __init__(self):
            self.columns, self.ended = [], False

        def put(self, tokens):
            assert tokens.shape == (2, 1) and not self.ended
            self.columns.append(tokens)

        def end(self):
            self.ended = True
    model.engine.scheduler.max_num_batched_tokens = 3          # the two prompts cannot share a step
    collect = Collect()
    out = model.sample(padded, sequence_length=9, start_ids=torch.tensor([2, 0]), top_k=1, streamer=collect)
    model.engine.scheduler.max_num_batched_tokens = 2048
    assert collect.ended and torch.equal(torch.cat(collect.columns, dim=1), out[:, 4:])
    assert out[0, 4:].tolist() == plain_opt.greedy(weights, cfg, [5, 9], 5)[2:]
    # other generation options from the next call on (base.py:761-766)
    from transformers_neuronx_amd.config import GenerationConfig
    model.update_generation_config(GenerationConfig(do_sample=False))
    out = model.sample(ids, sequence_length=12)
    assert out[0].tolist() == plain_opt.greedy(weights, cfg, ids[0].tolist(), 8)


def _toy_model(ops_kind, dtype, device):
    import toy_parts
    from transformers_neuronx_amd.cache import CacheManager
    from transformers_neuronx_amd.engine import DecoderModel, ModelRunner
    from transformers_neuronx_amd.kernels import make_ops
    from transformers_neuronx_amd.weights import TensorDict, random_tensors
    spec = toy_parts.toy_spec()
    model = DecoderModel(spec)
    tensors = random_tensors(model.param_decls(), spec.init_std, 3, dtype)    # stored as the engine computes
    ops = make_ops(ops_kind, dtype, device)
    model.load(TensorDict(tensors), ops, dtype, device)
    needs = model.cache_needs()
    cache = CacheManager(needs, 16, 12, 4, dtype, device)
    return ModelRunner(model, cache, ops), tensors


def run_toy_model(ops_kind, dtype, device, tol):
    import toy_parts
    runner, tensors = _toy_model(ops_kind, dtype, device)
    cache = runner.cache
    assert set(cache.groups) == {"full", "window24"}
    assert len(cache.groups["full"].cache_ids) == 2 and len(cache.groups["window24"].cache_ids) == 1
    states = [c for c in cache.caches.values() if c.state]
    assert len(states) == 2                                    # the layer named twice has a state per call
    requests = _requests(300, [70, 33, 100], 8)
    expected = {rid: toy_parts.toy_plain_logits(tensors, toks) for rid, toks in requests.items()}
    for steps, place in (schedules.whole(requests), schedules.portions(requests),
                         schedules.mixed(requests, max_tokens=192, page=16, seed=2, tail=8, max_live=3)):
        for rec in steps:
            logits = runner.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in rec["entries"]])
            for row in range(logits.shape[0]):
                rid, pos = place[(rec["step"], row)]
                want = expected[rid][pos]
                err = float((logits[row].cpu() - want).abs().max() / want.abs().max())
                assert err < tol, (rec["step"], rid, pos, err)
            for rid in rec["end"]:
                runner.finish(rid)
            cache.check()
        assert not cache.requests


def test_toy_parts_on_the_host():
    run_toy_model("reference", torch.float32, "cpu", 2e-5)


def run_toy_routed_model(ops_kind, dtype, device, tol):
    """A feed-forward that routes tokens to experts and a position encoding of another kind, both defined
    in the tests, built and stepped under every way of cutting without a change to the framework."""
    import toy_parts
    from transformers_neuronx_amd.cache import CacheManager
    from transformers_neuronx_amd.engine import DecoderModel, ModelRunner
    from transformers_neuronx_amd.kernels import make_ops
    from transformers_neuronx_amd.weights import TensorDict, random_tensors
    spec = toy_parts.toy_spec_routed()
    model = DecoderModel(spec)
    assert not model.recordable                                 # toy parts do not claim to be replayable
    tensors = random_tensors(model.param_decls(), spec.init_std, 5, dtype)    # stored as the engine computes
    ops = make_ops(ops_kind, dtype, device)
    model.load(TensorDict(tensors), ops, dtype, device)
    runner = ModelRunner(model, CacheManager(model.cache_needs(), 16, 12, 4, dtype, device), ops, use_graphs=True)
    requests = _requests(211, [70, 33, 100], 9)
    expected = {rid: toy_parts.toy_routed_plain_logits(tensors, toks) for rid, toks in requests.items()}
    for steps, place in (schedules.whole(requests), schedules.portions(requests),
                         schedules.mixed(requests, max_tokens=192, page=16, seed=2, tail=8, max_live=3)):
        for rec in steps:
            logits = runner.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in rec["entries"]])
            for row in range(logits.shape[0]):
                rid, pos = place[(rec["step"], row)]
                want = expected[rid][pos]
                err = float((logits[row].cpu() - want).abs().max() / want.abs().max())
                assert err < tol, (rec["step"], rid, pos, err)
            for rid in rec["end"]:
                runner.finish(rid)
            runner.cache.check()
        assert not runner.cache.requests


def test_toy_routed_parts_on_the_host():
    run_toy_routed_model("reference", torch.float32, "cpu", 2e-5)


def run_toy_rotating_model(ops_kind, dtype, device, tol, in_the_projection=False):
    """Attention whose queries and keys are turned by an encoding defined in the tests, a norm that brings a
    kernel of its own, tensor names of its own: built from the registries and stepped under every way of
    cutting, without a change to the framework."""
    import toy_parts
    from transformers_neuronx_amd.cache import CacheManager
    from transformers_neuronx_amd.engine import DecoderModel, ModelRunner
    from transformers_neuronx_amd.kernels import make_ops
    from transformers_neuronx_amd.weights import TensorDict, random_tensors
    # `in_the_projection`: the encoding hands over its pairwise tables, the projection's launch turns queries and
    # keys, every part can be replayed from a recording (the layer with Python loops is left out of that model)
    spec = toy_parts.toy_spec_rotating(tables=in_the_projection, latent_layer=not in_the_projection)
    model = DecoderModel(spec)
    tensors = random_tensors(model.param_decls(), spec.init_std, 6, dtype)    # stored as the engine computes
    assert "blocks.2.attn.wk.weight" in tensors and tensors["blocks.0.attn.wk.weight"].shape == (32, 96)
    ops = make_ops(ops_kind, dtype, device)
    model.load(TensorDict(tensors), ops, dtype, device)
    assert model.recordable == in_the_projection
    runner = ModelRunner(model, CacheManager(model.cache_needs(), 16, 12, 4, dtype, device), ops, use_graphs=True)
    if not in_the_projection:
        assert tensors["blocks.1.attn.down.weight"].shape == (24, 96)
        # the latent mixer's pages are of its own shape, in the same group (same page numbers) as the attention's
        shapes = {cid: {k: tuple(v.shape) for k, v in c.pages.items()} for cid, c in runner.cache.caches.items()}
        assert shapes[1] == {"z": (12, 16, 24)} and shapes[0] == {"k": (12, 1, 16, 32), "v": (12, 1, 32, 16)}
    assert list(runner.cache.groups) == ["full"]
    requests = _requests(157, [70, 33, 100], 10)
    expected = {rid: toy_parts.toy_rotating_plain_logits(tensors, toks, latent_layer=not in_the_projection)
                for rid, toks in requests.items()}
    for steps, place in (schedules.whole(requests), schedules.portions(requests),
                         schedules.mixed(requests, max_tokens=192, page=16, seed=2, tail=8, max_live=3)):
        for rec in steps:
            logits = runner.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in rec["entries"]])
            for row in range(logits.shape[0]):
                rid, pos = place[(rec["step"], row)]
                want = expected[rid][pos]
                err = float((logits[row].cpu() - want).abs().max() / want.abs().max())
                assert err < tol, (rec["step"], rid, pos, err)
            for rid in rec["end"]:
                runner.finish(rid)
            runner.cache.check()
        assert not runner.cache.requests
    return runner


def test_toy_rotating_parts_on_the_host():
    run_toy_rotating_model("reference", torch.float32, "cpu", 2e-5)
    run_toy_rotating_model("reference", torch.float32, "cpu", 2e-5, in_the_projection=True)


def test_toy_rotation_counts_distances_only():
    """What pins the toy's plain form: with every position shifted by the same amount the logits stay; with
    the keys turned the other way (a wrong sign) they would not."""
    import toy_parts
    from transformers_neuronx_amd.engine import DecoderModel
    from transformers_neuronx_amd.weights import random_tensors
    spec = toy_parts.toy_spec_rotating()
    tensors = random_tensors(DecoderModel(spec).param_decls(), spec.init_std, 6, torch.float32)
    toks = _requests(157, [40], 3)["r0"]
    a = toy_parts.toy_rotating_plain_logits(tensors, toks)
    b = toy_parts.toy_rotating_plain_logits(tensors, toks, first_position=37)
    assert float((a - b).abs().max() / a.abs().max()) < 1e-4
    c = toy_parts.toy_rotating_plain_logits(tensors, toks[::-1])
    assert float((a - c).abs().max() / a.abs().max()) > 1e-2       # and positions do matter


def test_model_without_the_norm_before_the_head(tmp_path):
    """`_remove_final_layer_norm` of an OPT config.json: the engine and the plain implementation both leave
    the norm out, and a model that keeps it answers differently."""
    from safetensors.torch import load_file
    from transformers_neuronx_amd.weights import write_random_model
    from conftest import TINY_A
    raw = dict(TINY_A, _remove_final_layer_norm=True)
    folder = write_random_model(OPTConfig.from_dict(raw), str(tmp_path / "m"), 3, dtype="float32")
    weights = load_file(folder + "/model.safetensors")
    toks = _requests(512, [23], 1)["r0"]
    runner, _ = _runner(folder, 64)
    got = runner.step([StepEntry("a", toks, list(range(len(toks))))])
    want = plain_opt.forward_logits(weights, raw, toks)
    assert float((got - want).abs().max()) < 1e-5
    g = torch.Generator().manual_seed(0)
    with_norm = dict(weights)
    with_norm["model.decoder.final_layer_norm.weight"] = 1 + 0.5 * torch.randn(64, generator=g)
    with_norm["model.decoder.final_layer_norm.bias"] = torch.randn(64, generator=g)
    other = plain_opt.forward_logits(with_norm, TINY_A, toks)
    assert float((other - want).abs().max()) > 1e-2


def test_tapped_tensors_are_the_plain_intermediates(tiny_folders):
    """Inside a debug context a step keeps the tensors the model taps: the embedded tokens, the stream after
    every layer call, the stream between a block's halves, the logits. They are the plain implementation's."""
    from transformers_neuronx_amd import debug
    folder, cfg, weights = tiny_folders["A"]
    toks = _requests(cfg["vocab_size"], [19], 2)["r0"]
    runner, _ = _runner(folder, 64)
    assert not debug.active()
    with debug.debug_context() as kept:
        assert debug.active()
        runner.step([StepEntry("a", toks, [len(toks) - 1])])
    assert not debug.active()
    assert list(kept) == ["embedding", "after_mixer", "call0.layer0", "after_mixer#2", "call1.layer1", "logits"]
    x = plain_opt.embed(torch.tensor(toks), weights, cfg)
    assert float((kept["embedding"] - x).abs().max()) < 1e-6
    for i in range(2):
        x = plain_opt.block(x, weights, cfg, i)
        assert float((kept[f"call{i}.layer{i}"] - x).abs().max()) < 1e-5
    assert float((kept["logits"][0] - plain_opt.head(x, weights, cfg)[-1]).abs().max()) < 1e-5
    # outside a context nothing is kept, and the step is the same
    again = runner.step([StepEntry("b", toks, [len(toks) - 1])])
    assert torch.equal(again, kept["logits"])


def test_percentiles_of_the_benchmark_report():
    from transformers_neuronx_amd.opt.demo import percentile
    values = [5.0, 1.0, 4.0, 2.0, 3.0]
    assert [percentile(values, q) for q in (0, 50, 90, 95, 99, 100)] == [1.0, 3.0, 5.0, 5.0, 5.0, 5.0]
    assert percentile([7.0], 50) == 7.0 and percentile(list(range(10)), 50) == 5 and percentile(list(range(10)), 96) == 9


def test_a_step_planner_of_the_tests_rides_in_the_steps_integers(tiny_folders):
    """A part that brings a kernel of its own can bring what that kernel launches by: a planner registered
    from outside adds its int32 arrays to the one buffer of integers a step sends, beside the attention
    kernels' own plan, and the model runs as before."""
    import numpy as np
    from transformers_neuronx_amd.engine import register_step_planner, unregister_step_planner

    def even_runs(run_lens, cached, page_size):
        chosen = np.nonzero(run_lens % 2 == 0)[0].astype(np.int32)
        return {"toy_even_runs": chosen, "toy_totals": (run_lens + cached).astype(np.int32)}, {"toy_count": len(chosen)}

    folder, cfg, weights = tiny_folders["A"]
    toks = _requests(cfg["vocab_size"], [6, 9, 4], 5)
    want = {rid: plain_opt.forward_logits(weights, cfg, t)[-1] for rid, t in toks.items()}
    register_step_planner("toy", even_runs)
    try:
        runner, _ = _runner(folder, 128)
        logits = runner.step([StepEntry(rid, t, [len(t) - 1]) for rid, t in toks.items()])
        ctx = runner._last_ctx
        assert ctx.plan["toy_even_runs"].tolist() == [0, 2] and ctx.plan["toy_totals"].tolist() == [6, 9, 4]
        assert ctx.plan_host["toy_count"] == 2
        # beside the plan that the model's attention mixers bring
        assert ctx.plan["decode_runs"].numel() == 0 and ctx.plan["tile_run"].tolist() == [1, 0, 2]     # the longest run first
        for i, rid in enumerate(toks):
            assert float((logits[i] - want[rid]).abs().max()) < 1e-5
    finally:
        unregister_step_planner("toy")
    runner, _ = _runner(folder, 128)
    runner.step([StepEntry("a", toks["r0"], [0])])
    assert "toy_even_runs" not in runner._last_ctx.plan


def _plain_without_repeats(weights, cfg, prompt, n_new, size, banned_token=None):
    toks = list(prompt)
    for _ in range(n_new):
        row = plain_opt.forward_logits(weights, cfg, toks)[-1].clone()
        if banned_token is not None:
            row[banned_token] = float("-inf")
        row[plain_opt.banned_by_ngrams(toks, size)] = float("-inf")
        toks.append(int(row.argmax()))
    return toks[len(prompt):]


@pytest.mark.parametrize("run_ahead", [False, True])
def test_no_run_of_tokens_twice(tiny_folders, run_ahead):
    """`no_repeat_ngram_size` (sampling.py:267-309): the greedy path of the narrow-weights model repeats one
    token; with the ban no run of n tokens comes twice, the tokens are the plain implementation's under the same
    ban, requests with and without it share steps, and a request put back and computed again keeps its path."""
    folder, cfg, weights = tiny_folders["A"]
    runner, ecfg = _runner(folder, max_tokens=64, run_ahead=run_ahead)
    engine = LLMEngine(runner, ecfg)
    prompts = [[5, 9, 200, 31, 9, 200], [7, 7, 100, 3], [11, 12]]
    sizes = [2, 3, 0]
    params = [SamplingParams(max_new_tokens=20, do_sample=False, ignore_eos=True, no_repeat_ngram_size=n) for n in sizes]
    outs = engine.generate(prompts, params)
    assert engine.scheduler.num_preemptions > 0            # four pages of 16 for three requests of up to 26 tokens
    for prompt, out, n in zip(prompts, outs, sizes):
        want = _plain_without_repeats(weights, cfg, prompt, 20, n) if n else plain_opt.greedy(weights, cfg, prompt, 20)[len(prompt):]
        assert out == want, (n, out, want)
        if n:
            whole = prompt + out
            runs = [tuple(whole[i:i + n]) for i in range(len(prompt) - n + 1, len(whole) - n + 1)]
            seen = {tuple(whole[i:i + n]) for i in range(len(prompt) - n + 1)}
            for r in runs:
                assert r not in seen, r
                seen.add(r)
    assert len(set(outs[2])) < 4                           # the row without the ban does repeat itself
    with pytest.raises(ValueError, match="strictly positive integer"):
        SamplingParams(no_repeat_ngram_size=-2)


def test_sample_takes_the_ngram_ban(tiny_folders):
    from transformers_neuronx_amd import OPTForSampling
    folder, cfg, weights = tiny_folders["A"]
    model = OPTForSampling.from_pretrained(folder, batch_size=2, amp="f32", n_positions=32, kernels="reference",
                                           device="cpu", page_size=16).to_neuron()
    ids = torch.tensor([[5, 9, 200, 31], [7, 7, 100, 3]])
    out = model.sample(ids, sequence_length=16, top_k=1, no_repeat_ngram_size=2)
    eos = cfg.get("eos_token_id", 2)
    for b in range(2):
        assert out[b, 4:].tolist() == _plain_without_repeats(weights, cfg, ids[b].tolist(), 12, 2, banned_token=eos)


@pytest.mark.parametrize("run_ahead", [False, True])
def test_a_request_taken_out_midway(tiny_folders, run_ahead):
    """`abort_request` between two steps: the request reports nothing more (a step under way may still hold
    a token for it), what it held is free at once, and the others go on as if it had never been there."""
    folder, cfg, weights = tiny_folders["B"]
    runner, ecfg = _runner(folder, max_tokens=256, run_ahead=run_ahead)
    engine = LLMEngine(runner, ecfg)
    prompts = [[5, 9, 200, 31], [7, 7, 100, 3, 8, 15], [11, 12, 13]]
    params = SamplingParams(max_new_tokens=12, do_sample=False, ignore_eos=True)
    ids = [engine.add_request(p, params) for p in prompts]
    late = engine.add_request([4, 4, 4], params)           # one that is still waiting when it is taken out
    engine.scheduler.max_num_seqs = 3
    got = {i: [] for i in ids + [late]}
    gone = None
    for step in range(200):
        if not engine.has_work:
            break
        for out in engine.step():
            assert out.req_id != ids[1] or gone is None, "a token after the request was taken out"
            got[out.req_id].append(out.token)
        if step == 4:
            assert runner.cache.has(ids[1])
            gone = engine.abort_request(ids[1])
            engine.abort_request(late)
            assert gone.finished and gone.finish_reason == "aborted" and not runner.cache.has(ids[1])
            assert gone.output == got[ids[1]] and 0 < len(gone.output) < 12
            runner.cache.check()
    assert not engine.has_work and not runner.cache.requests
    for i in (0, 2):
        assert got[ids[i]] == plain_opt.greedy(weights, cfg, prompts[i], 12)[len(prompts[i]):]
    assert got[late] == [] and ids[1] not in engine.requests
    with pytest.raises(KeyError):
        engine.abort_request("nobody")
    # a request that has ended by its length while its last token is still in a step under way: taken out, it
    # keeps no placeholder and reports nothing more; handed over in the ordinary way, only once the token is there
    for take_out in (True, False):
        rid = engine.add_request(prompts[0], SamplingParams(max_new_tokens=2, do_sample=False, ignore_eos=True))
        seen = []
        while not engine.requests[rid].finished:
            seen += [o.token for o in engine.step()]
        want = plain_opt.greedy(weights, cfg, prompts[0], 2)[len(prompts[0]):]
        if take_out:
            req = engine.abort_request(rid)
            assert PENDING not in req.output and req.output == seen and req.finish_reason == "length"
            while engine.has_work:
                assert engine.step() == []
        else:
            if run_ahead:
                assert PENDING in engine.requests[rid].output
                with pytest.raises(ValueError, match="under way"):
                    engine.pop_request(rid)
            while engine.has_work:
                seen += [o.token for o in engine.step()]
            assert engine.pop_request(rid).output == seen == want
        assert not runner.cache.requests


def test_several_tokens_end_a_request(tiny_folders):
    """`eos_token_id` as a list (sampling.py:319-322): the request ends at the first of them it generates, and
    with `ban_eos` none of them is ever chosen."""
    folder, cfg, weights = tiny_folders["B"]
    runner, ecfg = _runner(folder, max_tokens=128)
    engine = LLMEngine(runner, ecfg)
    prompt = [5, 9, 200, 31]
    free = plain_opt.greedy(weights, cfg, prompt, 12)[len(prompt):]
    stops = [free[6], free[3], 999]
    out = engine.generate([prompt], SamplingParams(max_new_tokens=12, do_sample=False, eos_token_id=stops))[0]
    assert out == free[:free.index(free[3]) + 1]
    out = engine.generate([prompt], SamplingParams(max_new_tokens=12, do_sample=False, eos_token_id=stops, ban_eos=True,
                                                   ignore_eos=True))[0]
    toks = list(prompt)
    for _ in range(12):
        row = plain_opt.forward_logits(weights, cfg, toks)[-1].clone()
        row[stops] = float("-inf")
        toks.append(int(row.argmax()))
    assert out == toks[len(prompt):] and not set(out) & set(stops)


def test_host_loops_by_their_names(tiny_folders):
    """`sampling.simple_sample` and `sampling.sample_greedy` (sampling.py:26-30, :108-128) as functions of a
    model: greedy with top_k 1, the scores of every step on request, another end-of-sequence token than the
    configuration's."""
    from transformers_neuronx_amd import OPTForSampling
    from transformers_neuronx_amd.sampling import sample_greedy, simple_sample
    folder, cfg, weights = tiny_folders["B"]
    model = OPTForSampling.from_pretrained(folder, batch_size=2, amp="f32", n_positions=32, kernels="reference",
                                           device="cpu", page_size=16).to_neuron()
    ids = torch.tensor([[5, 9, 200, 31], [7, 7, 100, 3]])
    free = [plain_opt.greedy(weights, cfg, ids[b].tolist(), 8) for b in range(2)]
    assert sample_greedy(model, ids, sequence_length=12).tolist() == free
    banned = free[0][6]                                        # a token the free path takes
    tokens, scores = simple_sample(model, ids, None, 12, eos_token_id=banned, top_k=1, output_scores=True)
    assert len(scores) == 8 and scores[0].shape == (2, cfg["vocab_size"]) and bool(torch.isinf(scores[3][:, banned]).all())
    assert banned not in tokens[0, 4:].tolist() and tokens[0, :6].tolist() == free[0][:6]
    row = plain_opt.forward_logits(weights, cfg, ids[0].tolist())[-1]
    keep = [i for i in range(cfg["vocab_size"]) if i != banned]
    torch.testing.assert_close(scores[0][0][keep], row[keep], rtol=1e-4, atol=1e-5)
    assert model.config.eos_token_id == cfg.get("eos_token_id", 2) and model.engine.logits_hook is None

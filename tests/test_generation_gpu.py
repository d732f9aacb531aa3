"""The scheduler and the engine on the HIP kernels against the plain implementation: generation with so
few pages that requests are put back and computed again, with steps started ahead of their tokens, with
recorded decode steps, portions of prompts, sampled tokens and requests that end late."""
import pytest
import torch

import plain_opt

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _prompts(vocab, lengths, seed):
    g = torch.Generator().manual_seed(seed)
    return [torch.randint(3, vocab, (n,), generator=g).tolist() for n in lengths]


def _engine(folder, dtype, **kw):
    from transformers_neuronx_amd.config import EngineConfig
    from transformers_neuronx_amd.engine.engine import LLMEngine
    from transformers_neuronx_amd.engine.factory import runner_from_folder
    cfg = EngineConfig(dtype=dtype, kernels="hip", device=DEV, **kw)
    runner = runner_from_folder(folder, cfg)
    return LLMEngine(runner, cfg), runner


def _plain_sampled(weights, cfg, prompt, sp, n_new):
    """The plain implementation's tokens for one request, and for every draw how far the random number lay
    from the nearest boundary between two tokens (a draw that close may fall either way in another
    arithmetic)."""
    toks, margins = list(prompt), []
    for n in range(n_new):
        row = plain_opt.forward_logits(weights, cfg, toks)[-1]
        if sp.greedy:
            top2 = row.topk(2).values
            margins.append(float(top2[0] - top2[1]) / float(row.abs().max()))
            toks.append(int(row.argmax()))
            continue
        u = plain_opt.philox_uniform(sp.seed, n)
        values, indices = plain_opt.filter_top_k_top_p(row / sp.temperature, sp.top_k or None, sp.top_p,
                                                       sp.min_tokens_to_keep)
        order = torch.argsort(indices)
        cum = torch.cumsum(torch.softmax(values[order].double(), -1), -1)
        margins.append(float((cum - u).abs().min()))
        toks.append(plain_opt.sample_row(row, u, sp.top_k or None, sp.top_p, sp.temperature, sp.min_tokens_to_keep))
    return toks[len(prompt):], margins


def _check_exact(outs, prompts, params, weights, cfg):
    for out, prompt, sp in zip(outs, prompts, params):
        want, margins = _plain_sampled(weights, cfg, prompt, sp, len(out))
        if out != want:
            first = next(i for i, (a, b) in enumerate(zip(out, want)) if a != b)
            # only a draw on a boundary (or two best logits a rounding apart) may differ
            assert margins[first] < 1e-5, (first, out, want, margins[first])


# Two workloads: three short prompts decoded greedily, and five prompts taken in portions of 32 beside
# decoding requests, drawn at temperature 0.8 from fixed seeds.
WORKLOADS = {
    "A": dict(lengths=[5, 17, 31], new=16, chunk=None, temperature=0.0),
    "B": dict(lengths=[1, 9, 40, 77, 120], new=14, chunk=32, temperature=0.8),
    # the model with the norm before the head, its prompts in portions: steps that ask nothing of the head
    "C": dict(lengths=[3, 64, 65, 150], new=10, chunk=32, temperature=0.0),
}


@pytest.mark.parametrize("name", ["A", "B", "C"])
@pytest.mark.parametrize("run_ahead", [False, True])
def test_generation_with_few_pages_float32(tiny_folders, name, run_ahead):
    from transformers_neuronx_amd.sampling import SamplingParams
    folder, cfg, weights = tiny_folders[name]
    w = WORKLOADS[name]
    prompts = _prompts(cfg["vocab_size"], w["lengths"], 31)
    params = [SamplingParams(max_new_tokens=w["new"], do_sample=w["temperature"] > 0,
                             temperature=w["temperature"] or 1.0, seed=100 + i, ignore_eos=True)
              for i in range(len(prompts))]
    total = sum(w["lengths"]) + w["new"] * len(prompts)
    roomy = -(-total // 16) * 16 + 16 * len(prompts)
    # pages for a little more than the longest request alone: the others are put back again and again
    tight = -(-(max(w["lengths"]) + w["new"]) // 16) * 16 + 32
    results = {}
    for kind, max_tokens in (("roomy", roomy), ("tight", tight)):
        engine, runner = _engine(folder, "float32", page_size=16, max_tokens=max_tokens, max_num_seqs=4,
                                 max_num_batched_tokens=48, chunk_size=w["chunk"], run_ahead=run_ahead,
                                 use_graphs=True)
        outs = engine.generate(prompts, params)
        runner.cache.check()
        assert not runner.cache.requests and not engine.requests
        results[kind] = outs
        if kind == "roomy":
            assert engine.scheduler.num_preemptions == 0 and runner.graph_replays > 0
        else:
            assert engine.scheduler.num_preemptions > 0
    assert results["roomy"] == results["tight"]
    _check_exact(results["tight"], prompts, params, weights, cfg)


def test_every_way_of_choosing_a_token_in_one_batch_float32(tiny_folders):
    """Requests that differ in how their tokens are chosen, side by side in every step: greedy, top-p alone, a
    top-k beyond what the sampler gathers with top-p, a small top-k alone, a top-p so tight that the least
    number of tokens to keep decides, and the plain softmax. Each takes its own way through the sampling
    kernel; all are the plain implementation's tokens."""
    from transformers_neuronx_amd.sampling import SamplingParams
    folder, cfg, weights = tiny_folders["B"]
    prompts = _prompts(cfg["vocab_size"], [7, 30, 2, 55, 18, 41], 77)
    params = [SamplingParams(max_new_tokens=20, do_sample=False, ignore_eos=True),
              SamplingParams(max_new_tokens=20, temperature=1.1, top_p=0.7, seed=11, ignore_eos=True),
              SamplingParams(max_new_tokens=20, temperature=0.9, top_k=300, top_p=0.95, seed=12, ignore_eos=True),
              SamplingParams(max_new_tokens=20, temperature=1.4, top_k=5, seed=13, ignore_eos=True),
              SamplingParams(max_new_tokens=20, temperature=1.3, top_p=0.05, min_tokens_to_keep=4, seed=14,
                             ignore_eos=True),
              SamplingParams(max_new_tokens=20, temperature=0.7, seed=15, ignore_eos=True)]
    engine, runner = _engine(folder, "float32", page_size=16, max_tokens=640, max_num_seqs=6,
                             max_num_batched_tokens=64, use_graphs=True)
    outs = engine.generate(prompts, params)
    runner.cache.check()
    assert not runner.cache.requests and not engine.requests
    assert all(len(o) == 20 for o in outs)
    _check_exact(outs, prompts, params, weights, cfg)


@pytest.mark.parametrize("prompts_first", [False, True])
def test_late_end_of_sequence_and_arrivals_float32(tiny_folders, prompts_first):
    """Requests that stop at a token they generate (found out a step late when steps run ahead), others
    that arrive while the first ones run, few pages, top-k and top-p: every token is reported once and the
    tokens are the plain implementation's."""
    from transformers_neuronx_amd.sampling import SamplingParams
    folder, cfg, weights = tiny_folders["B"]
    prompts = _prompts(cfg["vocab_size"], [3, 9, 40, 77, 20, 5], 8)
    free = [SamplingParams(max_new_tokens=12, do_sample=False, ignore_eos=True),
            SamplingParams(max_new_tokens=12, temperature=0.9, top_k=20, top_p=0.9, seed=4, ignore_eos=True)] * 3
    first = {}
    for i, (p, sp) in enumerate(zip(prompts, free)):
        first[i] = _plain_sampled(weights, cfg, p, sp, 12)
    # each request stops at the token it generates fifth (or at that token's first appearance)
    stopping = [SamplingParams(max_new_tokens=12, do_sample=sp.do_sample, temperature=sp.temperature, top_k=sp.top_k,
                               top_p=sp.top_p, seed=sp.seed, eos_token_id=first[i][0][4])
                for i, sp in enumerate(free)]
    want = [first[i][0][:first[i][0].index(first[i][0][4]) + 1] for i in range(6)]
    for run_ahead in (False, True):
        engine, runner = _engine(folder, "float32", page_size=16, max_tokens=160, max_num_seqs=4,
                                 max_num_batched_tokens=32, run_ahead=run_ahead, prompts_first=prompts_first)
        seen, ends = {}, {}
        ids = [engine.add_request(p, sp) for p, sp in zip(prompts[:4], stopping[:4])]
        calls = 0
        while engine.has_work:
            for out in engine.step():
                assert out.req_id not in ends, "a token after the last one"
                seen.setdefault(out.req_id, []).append(out.token)
                if out.finished:
                    ends[out.req_id] = out.finish_reason
            calls += 1
            if calls == 3:
                ids += [engine.add_request(p, sp) for p, sp in zip(prompts[4:], stopping[4:])]
            assert calls < 1000
        runner.cache.check()
        assert not runner.cache.requests
        outs = [seen[i] for i in ids]
        assert all(ends[i] == "eos" for i in ids)
        for i in range(6):
            if outs[i] != want[i]:
                k = next(j for j, (a, b) in enumerate(zip(outs[i], want[i])) if a != b)
                assert first[i][1][k] < 1e-5, (i, outs[i], want[i])


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_generation_with_few_pages_bfloat16(tiny_folders_bf16, name):
    """In bfloat16 a choice may part from the float32 one where two logits are a rounding apart: every
    greedy token must be within the rounding of the best one under the plain implementation, given the
    tokens before it; and the tokens do not depend on whether pages were scarce."""
    from transformers_neuronx_amd.sampling import SamplingParams
    folder, cfg, weights = tiny_folders_bf16[name]
    w = WORKLOADS[name]
    prompts = _prompts(cfg["vocab_size"], w["lengths"], 5)
    params = [SamplingParams(max_new_tokens=w["new"], do_sample=False, ignore_eos=True) for _ in prompts]
    tight = -(-(max(w["lengths"]) + w["new"]) // 16) * 16 + 32
    for max_tokens in (1024, tight):
        engine, runner = _engine(folder, "bfloat16", page_size=16, max_tokens=max_tokens, max_num_seqs=4,
                                 max_num_batched_tokens=48, chunk_size=w["chunk"])
        outs = engine.generate(prompts, params)
        runner.cache.check()
        assert (engine.scheduler.num_preemptions > 0) == (max_tokens == tight)
        allowed = []
        for prompt, out in zip(prompts, outs):
            toks = prompt + out
            logits = plain_opt.forward_logits(weights, cfg, toks[:-1])
            for pos in range(len(prompt) - 1, len(toks) - 1):
                row = logits[pos]
                slack = 3e-2 * float(row.abs().max())
                assert float(row.max() - row[toks[pos + 1]]) <= slack, (pos, toks[pos + 1])
                allowed.append(int((row.max() - row <= slack).sum()))
        # and that says something: of the hundreds of tokens of the vocabulary one or two pass at a place
        assert sum(allowed) / len(allowed) < 3, sum(allowed) / len(allowed)


def test_no_run_of_tokens_twice_on_the_gpu(tiny_folders):
    """`no_repeat_ngram_size` through the HIP sampler's ban of (row, token) pairs, beside requests without it,
    with few pages and recorded decode steps: the plain implementation's tokens under the same ban."""
    from transformers_neuronx_amd.sampling import SamplingParams
    folder, cfg, weights = tiny_folders["A"]
    prompts = _prompts(cfg["vocab_size"], [6, 17, 3], 8)
    sizes = [2, 0, 3]
    params = [SamplingParams(max_new_tokens=24, do_sample=False, ignore_eos=True, no_repeat_ngram_size=n) for n in sizes]
    engine, runner = _engine(folder, "float32", page_size=16, max_tokens=80, max_num_seqs=4, use_graphs=True)
    outs = engine.generate(prompts, params)
    runner.cache.check()
    assert engine.scheduler.num_preemptions > 0
    for prompt, out, n in zip(prompts, outs, sizes):
        toks = list(prompt)
        for _ in range(24):
            row = plain_opt.forward_logits(weights, cfg, toks)[-1].clone()
            if n:
                row[plain_opt.banned_by_ngrams(toks, n)] = float("-inf")
            toks.append(int(row.argmax()))
        assert out == toks[len(prompt):], (n, out, toks[len(prompt):])
    # the kernel alone: pairs out of range touch nothing
    from transformers_neuronx_amd.kernels.hip import HipOps
    ops = HipOps(torch.float32, DEV)
    logits = torch.zeros(3, 10, device=DEV)
    rows = torch.tensor([0, 2, 2, 5, 1], dtype=torch.int32, device=DEV)
    toks = torch.tensor([4, 0, 9, 1, 10], dtype=torch.int32, device=DEV)
    ops.ban_pairs(logits, rows, toks)
    assert torch.isinf(logits).nonzero().tolist() == [[0, 4], [2, 0], [2, 9]]


@pytest.mark.parametrize("run_ahead", [False, True])
def test_a_request_taken_out_midway_on_the_gpu(tiny_folders, run_ahead):
    """`abort_request` while steps run ahead on the device: the slot and the pages it gives back go to a request
    that arrives afterwards, and every other request keeps the plain implementation's tokens."""
    from transformers_neuronx_amd.sampling import SamplingParams
    folder, cfg, weights = tiny_folders["A"]
    engine, runner = _engine(folder, "float32", page_size=16, max_tokens=96, max_num_seqs=3, run_ahead=run_ahead,
                             use_graphs=True)
    prompts = _prompts(cfg["vocab_size"], [9, 20, 5, 12], 3)
    params = SamplingParams(max_new_tokens=14, do_sample=False, ignore_eos=True)
    ids = [engine.add_request(p, params) for p in prompts[:3]]
    got = {}
    for step in range(300):
        if not engine.has_work:
            break
        for out in engine.step():
            got.setdefault(out.req_id, []).append(out.token)
        if step == 5:
            engine.abort_request(ids[1])
            ids.append(engine.add_request(prompts[3], params))     # takes the slot and pages just given back
    runner.cache.check()
    assert not engine.has_work and not runner.cache.requests
    for i in (0, 2, 3):
        assert got[ids[i]] == plain_opt.greedy(weights, cfg, prompts[i], 14)[len(prompts[i]):], i
    assert 0 < len(got[ids[1]]) < 14

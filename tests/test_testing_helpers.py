"""The package's own helpers for checking a model against a golden one, with the plain implementation as the
golden model: the three batch shapes of the reference's testing/data.py through `sample(top_k=1)`."""
import pytest
import torch

import plain_opt


def _golden(weights, cfg):
    eos = cfg.get("eos_token_id", 2)

    def follow(prompt, n):
        toks = list(prompt)
        for _ in range(n):
            row = plain_opt.forward_logits(weights, cfg, toks)[-1].clone()
            row[eos] = float("-inf")
            toks.append(int(row.argmax()))
        return toks[len(prompt):]
    return follow


def test_batch_builders():
    from transformers_neuronx_amd.testing import batch_all_lengths, batch_full_lengths, batch_varying_lengths
    g = torch.Generator().manual_seed(0)
    ids, mask, starts = batch_all_lengths(100, 5, pad_token_id=1, generator=g)
    assert ids.shape == (5, 5) and starts.tolist() == [0, 1, 2, 3, 4]
    assert torch.equal(mask, torch.ones(5, 5).triu().int()) and bool((ids[mask == 0] == 1).all())
    ids, mask, starts = batch_varying_lengths(100, 7, 6, generator=g)
    assert ids.shape == (7, 6) and bool((mask.sum(1) == 6 - starts).all()) and int(mask.sum(1).min()) >= 1
    assert bool((mask[:, -1] == 1).all())
    ids, mask, starts = batch_full_lengths(100, 3, 4, generator=g)
    assert bool(mask.all()) and not starts.any()


@pytest.mark.parametrize("shape", ["varying", "all", "full"])
def test_validate_on_the_host(tiny_folders, shape):
    from transformers_neuronx_amd import OPTForSampling
    from transformers_neuronx_amd.testing import batch_all_lengths, batch_full_lengths, batch_varying_lengths, validate
    folder, cfg, weights = tiny_folders["A"]
    g = torch.Generator().manual_seed(4)
    vocab = cfg["vocab_size"]
    inputs = {"varying": lambda: batch_varying_lengths(vocab, 4, 7, 1, g), "all": lambda: batch_all_lengths(vocab, 5, 1, g),
              "full": lambda: batch_full_lengths(vocab, 3, 6, 1, g)}[shape]()
    model = OPTForSampling.from_pretrained(folder, batch_size=inputs[0].shape[0], amp="f32", n_positions=32,
                                           kernels="reference", device="cpu", page_size=16)
    validate(_golden(weights, cfg), model, inputs, sequence_length=inputs[0].shape[1] + 6)
    # a golden model that disagrees is told apart
    with pytest.raises(AssertionError, match="row 0"):
        validate(lambda prompt, n: [3] * n, model, inputs, sequence_length=inputs[0].shape[1] + 2)


@pytest.mark.gpu
def test_validate_on_the_gpu(tiny_folders):
    from transformers_neuronx_amd import OPTForSampling
    from transformers_neuronx_amd.testing import batch_varying_lengths, validate
    folder, cfg, weights = tiny_folders["B"]
    inputs = batch_varying_lengths(cfg["vocab_size"], 4, 9, 1, torch.Generator().manual_seed(7))
    model = OPTForSampling.from_pretrained(folder, batch_size=4, amp="f32", n_positions=40, page_size=16)
    validate(_golden(weights, cfg), model, inputs, sequence_length=20)


def test_compare_precisions_on_the_host(tiny_folders):
    """The full-depth check's helper on the torch rendition of the kernels: an engine against itself differs
    nowhere, a bfloat16 engine held to the float32 engine's tokens differs by bfloat16 rounding and no more,
    and the logits the helper keeps are the plain implementation's at the followed tokens."""
    from transformers_neuronx_amd.config import EngineConfig
    from transformers_neuronx_amd.engine.engine import LLMEngine
    from transformers_neuronx_amd.engine.factory import runner_from_folder
    from transformers_neuronx_amd.testing import compare_logits, compare_precisions, greedy_logits
    folder, cfg, weights = tiny_folders["A"]

    def engine(dtype):
        ecfg = EngineConfig(dtype=dtype, kernels="reference", device="cpu", page_size=16, max_tokens=128, max_num_seqs=2,
                            cast_float32_weights=True)
        return LLMEngine(runner_from_folder(folder, ecfg), ecfg)

    wide, narrow = engine(torch.float32), engine(torch.bfloat16)
    prompt = torch.randint(3, 512, (21,), generator=torch.Generator().manual_seed(3)).tolist()
    same = compare_precisions(wide, wide, prompt, 6)
    assert same["rel"] == 0.0 and same["rows"] == same["same_argmax"] == same["clear_rows"] == same["clear_same"] == 6
    got = compare_precisions(wide, narrow, prompt, 6)
    assert 0.0 < got["rel"] < 3e-2 and got["allclose_rows"] == 6 and got["clear_same"] == got["clear_rows"]
    tokens, rows = greedy_logits(wide, prompt, 6)
    assert tokens == plain_opt.greedy(weights, cfg, prompt, 6)[len(prompt):]
    forced = [7, 9, 11, 13, 15, 17]
    tokens, rows = greedy_logits(narrow, prompt, 6, follow=forced)
    assert tokens == forced
    want = plain_opt.forward_logits(weights, cfg, prompt + forced[:-1])[len(prompt) - 1:]
    assert compare_logits(rows, want)["rel"] < 3e-2
    # a row whose winner changes where the golden one leads clearly is counted as such
    bad = want.clone()
    bad[2, int(want[2].argmax())] -= 1.0
    report = compare_logits(bad, want)
    assert report["same_argmax"] == 5 and report["max_abs_diff"] == 1.0 and report["clear_rows"] == report["clear_same"]
    top2 = want[2].topk(2).values
    assert float(top2[0] - top2[1]) < 2.0         # (the changed row is no clear one: its winner led by less than 2 x 1.0)

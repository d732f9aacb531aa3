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

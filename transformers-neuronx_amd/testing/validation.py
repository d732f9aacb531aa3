"""Greedy generation of a model against a golden one, token for token.

Reference: testing/validation.py:23-101 generates with an installed package's CPU model (`generate` with
`top_k=1` and as many new tokens as asked for, none fewer), with its own adapter to that package and with
`sample(top_k=1)`, and asserts equal ids. The golden model here is whatever the caller brings, as a function
from a prompt to its greedy continuation: this package reads no other package's model code.
"""
from typing import Callable, List, Sequence

import torch

Golden = Callable[[List[int], int], Sequence[int]]


def validate(golden: Golden, model, inputs, sequence_length: int, verbose: bool = False) -> None:
    """`inputs` is (input_ids, attention_mask, start_ids) as the builders of `testing.data` make them;
    `golden(prompt, n)` returns the n tokens that follow `prompt` when the largest logit is taken each time and
    the end-of-sequence token never (what `sample(top_k=1)` does, sampling.py:143-144). Raises
    AssertionError where a row of `model.sample` differs."""
    input_ids, attention_mask, start_ids = inputs
    batch, context = input_ids.shape
    new = sequence_length - context
    if not model.is_compiled():
        model.to_neuron()
    model.reset()
    actual = model.sample(input_ids, sequence_length=sequence_length, start_ids=start_ids, top_k=1)
    if verbose:
        print("Input Ids:", input_ids, "Start Ids:", start_ids, "Result (Sample):", actual, sep="\n")
    assert tuple(actual.shape) == (batch, sequence_length), f"sample returned {tuple(actual.shape)}"
    assert torch.equal(actual[:, :context], input_ids), "sample changed the prompts"
    for b in range(batch):
        prompt = input_ids[b, int(start_ids[b]):].tolist()
        expected = [int(t) for t in golden(prompt, new)]
        got = actual[b, context:].tolist()
        assert got == expected, f"row {b} (prompt of {len(prompt)} tokens): generated {got}, the golden model {expected}"

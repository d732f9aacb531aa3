"""Batches of prompts padded on the left, as (input_ids, attention_mask, start_ids): row b's prompt is
`input_ids[b, start_ids[b]:]`, the mask is 1 over it and 0 over the padding in front.

Reference: testing/data.py:18-77 has the same three shapes. Here a generator can be handed in, so that a test
names its tokens by a seed, and the padding holds `pad_token_id` rather than whatever was drawn.
"""
from typing import Optional, Tuple

import torch

Batch = Tuple[torch.Tensor, torch.Tensor, torch.Tensor]


def _padded(vocab_size: int, starts: torch.Tensor, context_length: int, pad_token_id: int,
            generator: Optional[torch.Generator]) -> Batch:
    rows = starts.numel()
    ids = torch.randint(0, vocab_size, (rows, context_length), generator=generator)
    mask = (torch.arange(context_length)[None, :] >= starts[:, None]).to(torch.int32)
    return torch.where(mask.bool(), ids, torch.full_like(ids, pad_token_id)), mask, starts


def batch_varying_lengths(vocab_size: int, batch_size: int, context_length: int, pad_token_id: int = 0,
                          generator: Optional[torch.Generator] = None) -> Batch:
    """Rows that begin at places drawn at random (each keeps one token at least): lengths mixed and out of
    order, e.g. masks 001 / 011 / 001 / 111 (testing/data.py:18-37)."""
    starts = torch.randint(0, context_length, (batch_size,), generator=generator)
    return _padded(vocab_size, starts, context_length, pad_token_id, generator)


def batch_all_lengths(vocab_size: int, context_length: int, pad_token_id: int = 0,
                      generator: Optional[torch.Generator] = None) -> Batch:
    """One row of every length from `context_length` down to 1: masks 111 / 011 / 001 (testing/data.py:40-58)."""
    return _padded(vocab_size, torch.arange(context_length), context_length, pad_token_id, generator)


def batch_full_lengths(vocab_size: int, batch_size: int, context_length: int, pad_token_id: int = 0,
                       generator: Optional[torch.Generator] = None) -> Batch:
    """Rows without padding: that batching works at all (testing/data.py:61-77)."""
    return _padded(vocab_size, torch.zeros(batch_size, dtype=torch.int64), context_length, pad_token_id, generator)

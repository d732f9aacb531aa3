"""Helpers for checking a model against a golden one (reference: testing/validation.py, testing/data.py)."""
from .data import batch_all_lengths, batch_full_lengths, batch_varying_lengths  # noqa: F401
from .validation import validate  # noqa: F401
from .precision import compare_logits, compare_precisions, greedy_logits  # noqa: F401

"""What a request asks of the sampler."""
import operator
from dataclasses import dataclass
from typing import Optional, Sequence, Tuple, Union


@dataclass
class SamplingParams:
    """Per-request sampling options.

    The names and meanings follow the reference's host loops (sampling.py:131-180,
    :311-378) and its `GenerationConfig` (config.py:106-139):
    temperature  logits are divided by it before filtering (:337-338); 0 selects the
                 argmax, as does do_sample=False
    top_k        the k largest logits are kept (:151, :210-211); 0 keeps all
    top_p        of those, the shortest prefix in descending order whose softmax mass
                 reaches top_p (:213-249); 1.0 keeps all
    min_tokens_to_keep  neither filter leaves fewer tokens than this (:204-205, :232;
                 `top_p_min_tokens` of the `GenerationConfig`)
    seed         the request's own random stream: draw number n of the request uses the
                 counter n, whatever else is in the batch; None lets the engine give one
                 (its own seed plus the request's number of arrival)
    deterministic  every draw uses 0.5 in place of a random number (hlo.py:2455-2456)
    eos_token_id the token that ends the request, or a list of such tokens (sampling.py:319-322)
    ban_eos      the end-of-sequence token is never chosen (`scores[:, eos] = -inf`,
                 sampling.py:143-144, the OPT loop's behaviour)
    ignore_eos   generation does not stop at the end-of-sequence token
    no_repeat_ngram_size  n: no run of n tokens appears twice in the prompt and what follows it; a token
                 that would complete a run seen before gets the logit -inf before anything else is done
                 (sampling.py:267-309, :334-335); 0 switches it off
    max_time     seconds: the request ends after the first token that arrives later than this after it was
                 taken in (stopping_criteria.py:15-35, `MaxTimeCriteria`)
    max_new_tokens  the most tokens to generate
    """
    max_new_tokens: int = 16
    do_sample: bool = True
    temperature: float = 1.0
    top_k: int = 0
    top_p: float = 1.0
    seed: Optional[int] = 0
    min_tokens_to_keep: int = 1
    deterministic: bool = False
    eos_token_id: Optional[Union[int, Sequence[int]]] = None      # one token or several (sampling.py:319-322)
    ban_eos: bool = False
    ignore_eos: bool = False
    no_repeat_ngram_size: int = 0
    max_time: Optional[float] = None

    def __post_init__(self):
        if self.max_new_tokens < 0:
            raise ValueError("max_new_tokens must not be negative")
        if not isinstance(self.top_k, int) or self.top_k < 0:
            raise ValueError("top_k has to be a non-negative int (0 keeps all tokens).")
        if not 0.0 < float(self.top_p) <= 1.0:
            raise ValueError("top_p has to be a strictly positive float that less than or equal to 1.0.")
        if not isinstance(self.min_tokens_to_keep, int) or self.min_tokens_to_keep < 1:
            raise ValueError("min_tokens_to_keep has to be a positive int.")
        if self.no_repeat_ngram_size and (not isinstance(self.no_repeat_ngram_size, int) or self.no_repeat_ngram_size <= 0):
            raise ValueError(f"`ngram_size` has to be a strictly positive integer, but is {self.no_repeat_ngram_size}")
        if float(self.temperature) < 0:
            raise ValueError("temperature has to be a non-negative float (0 is greedy).")
        # one token or several, of any integer type (a numpy or tensor scalar too): settled here, not when
        # the first token is compared with it
        if self.eos_token_id is not None:
            try:
                self.eos_token_id = operator.index(self.eos_token_id)
            except TypeError:
                try:
                    self.eos_token_id = tuple(operator.index(t) for t in self.eos_token_id)
                except TypeError:
                    raise ValueError(f"eos_token_id has to be an integer or a sequence of integers, got "
                                     f"{self.eos_token_id!r}") from None

    @property
    def eos_ids(self) -> Tuple[int, ...]:
        """The tokens that end the request, as a tuple (empty: none does)."""
        if self.eos_token_id is None:
            return ()
        if isinstance(self.eos_token_id, int):
            return (self.eos_token_id,)
        return tuple(int(t) for t in self.eos_token_id)

    @property
    def greedy(self) -> bool:
        return (not self.do_sample) or self.temperature == 0.0 or self.top_k == 1

    @staticmethod
    def greedy_params(max_new_tokens: int, eos_token_id=None, ignore_eos=True) -> "SamplingParams":
        return SamplingParams(max_new_tokens=max_new_tokens, do_sample=False, eos_token_id=eos_token_id,
                              ignore_eos=ignore_eos)

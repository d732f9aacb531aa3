"""Settings of the engine that are not properties of a checkpoint.

`EngineConfig` is what the engine reads. `ContinuousBatchingConfig`,
`GenerationConfig` and `NeuronConfig` keep the reference's names and meanings of
options (config.py:73-139, :206-363) for the ones that have a counterpart on one
GPU, so that code written against the reference's API keeps working.
"""
from dataclasses import dataclass, field
from typing import List, Optional, Union

import torch

_DTYPES = {
    "float32": torch.float32, "f32": torch.float32, "fp32": torch.float32,
    "bfloat16": torch.bfloat16, "bf16": torch.bfloat16,
}


def parse_dtype(name) -> torch.dtype:
    """Compute dtype from the reference's `amp` names (dtypes.py:18-35) or torch's.
    float16 storage is served in bfloat16: the kernels have one 16-bit format."""
    if isinstance(name, torch.dtype):
        if name in (torch.float32, torch.bfloat16):
            return name
        if name == torch.float16:
            return torch.bfloat16
        raise ValueError(f"unsupported dtype {name}")
    key = str(name).lower()
    if key in ("f16", "fp16", "float16"):
        return torch.bfloat16
    if key not in _DTYPES:
        raise ValueError(f"unsupported dtype {name!r}; use one of {sorted(_DTYPES)}")
    return _DTYPES[key]


@dataclass
class ContinuousBatchingConfig:
    """Capacities for continuous batching, named as in config.py:73-103.

    `block_size`/`num_blocks` are the page size and page count of the cache
    (set there by `init_cache_engine`, :100-102)."""
    max_num_seqs: Optional[int] = None
    max_model_len: Optional[int] = None
    optimized_paged_attention: bool = True
    enable_chunked_prefill: bool = True
    block_size: Optional[int] = None
    num_blocks: Optional[int] = None
    batch_size_for_shared_caches: Optional[int] = None

    def __post_init__(self):
        if self.max_num_seqs is None:
            self.max_num_seqs = self.batch_size_for_shared_caches
        if self.max_num_seqs is None:
            raise ValueError("max_num_seqs (or batch_size_for_shared_caches) is required")
        self.batch_size_for_shared_caches = self.max_num_seqs

    def init_cache_engine(self, block_size, num_blocks):
        self.block_size = block_size
        self.num_blocks = num_blocks


@dataclass
class GenerationConfig:
    """Generation options, named as in config.py:106-139."""
    max_length: Optional[int] = None
    do_sample: bool = False
    top_k: int = 50
    top_p: float = 1.0
    top_p_min_tokens: int = 1
    global_top_k: Optional[int] = None
    eos_token_id: Optional[Union[int, List[int]]] = None
    temperature: float = 1.0
    dynamic: bool = False
    deterministic: bool = False
    per_batch_line: bool = False

    def __post_init__(self):
        # a list gives every batch line its own value (`per_batch_line`)
        self.top_p = [float(p) for p in self.top_p] if isinstance(self.top_p, (list, tuple)) else float(self.top_p)
        self.temperature = ([float(t) for t in self.temperature] if isinstance(self.temperature, (list, tuple))
                            else float(self.temperature))


class NeuronConfig:
    """The reference's bag of switches (config.py:206-363), by its keyword names.

    What means something on one GPU is kept: `continuous_batching` sizes the scheduler and the cache,
    `on_device_generation` makes `sample` draw with these generation options, `output_all_logits` makes
    `forward` return the logits of every position, `cast_logits_dtype` is always float32 here,
    `padding_side` and `on_device_embedding` are recorded. Switches that only choose a layout, a fusion or
    a way of splitting work over devices are taken and change nothing (the kernels have their own
    layouts; there is one device). Switches that would change what is computed and have no counterpart
    here (quantization, sparse attention, grouped queries for OPT, speculative heads, log-softmax scores)
    are refused unless left at the reference's default."""

    # keyword -> the reference's default; any value is taken and ignored
    _NO_EFFECT = dict(attention_layout="HSB", collectives_layout="HSB", cache_layout="SBH", fuse_qkv=False,
                      fuse_mlp=False, qkv_tiling=False, weight_tiling=False,
                      mlp_in_weight_tiling_permute_order=[1, 2, 0, 3], mlp_out_weight_tiling_permute_order=[1, 2, 0, 3],
                      sequence_parallel_norm=False, sequence_parallel_norm_threshold=2048, all_reduce_dtype=None,
                      attn_output_transposed=False, mlp_out_weight_transpose=False, compilation_worker_count=None,
                      duplicate_q_weight_sos=False, use_2d_cache_ids=False, lhs_aligned=False)
    # keyword -> the only value taken
    _REFUSED = dict(sparse_attn=None, quant=None, kv_cache_quant=None, group_query_attention=None,
                    bf16_rms_norm=False, log_softmax_scores=False, shard_over_sequence=False,
                    fused_rmsnorm_qkv=False, fused_rmsnorm_mlp=False, is_eagle_target=False, is_eagle_draft=False,
                    has_pre_attention_norm=True)

    def __init__(self, *, continuous_batching=None, on_device_generation=None, on_device_embedding: bool = True,
                 cast_logits_dtype: str = "float32", output_all_logits: bool = False, padding_side: str = "left",
                 **kwargs):
        if isinstance(continuous_batching, dict):
            continuous_batching = ContinuousBatchingConfig(**continuous_batching)
        if cast_logits_dtype != "float32":
            raise ValueError("logits are returned in float32; cast_logits_dtype must be 'float32'")
        if padding_side not in ("left", "right"):
            raise ValueError(f"padding_side must be 'left' or 'right', got {padding_side!r}")
        self.continuous_batching: Optional[ContinuousBatchingConfig] = continuous_batching
        self.on_device_generation: Optional[GenerationConfig] = on_device_generation
        self.on_device_embedding = on_device_embedding
        self.cast_logits_dtype = cast_logits_dtype
        self.output_all_logits = output_all_logits
        self.padding_side = padding_side
        for name, default in self._NO_EFFECT.items():
            setattr(self, name, kwargs.pop(name, default))
        for name, only in self._REFUSED.items():
            value = kwargs.pop(name, only)
            if value != only:
                raise ValueError(f"NeuronConfig({name}={value!r}) has no counterpart in this engine; "
                                 f"leave it at {only!r}")
            setattr(self, name, value)
        if kwargs:
            raise TypeError(f"NeuronConfig got unknown keywords {sorted(kwargs)}")


@dataclass
class EngineConfig:
    """What the engine is built with.

    dtype            compute and storage dtype: torch.bfloat16 or torch.float32
    page_size        tokens per cache page (a multiple of 16)
    num_pages        pages per cache group; None sizes the pool from `max_tokens`
                     or, failing that, from free device memory
    max_tokens       the most tokens live requests hold at a time
    max_num_seqs     the most live requests (slots of per-request state)
    max_num_batched_tokens   token budget of one step
    chunk_size       the most tokens of one prompt that one step takes (its portion); None: what is left
                     of the step's token budget
    max_model_len    longest request (prompt + generated); capped by the model
    kernels          "hip" (the product path) or "reference" (the plain torch
                     rendition of every kernel, for debugging on any device;
                     never chosen by itself)
    prompts_first    scheduling: take in every waiting prompt before the next decode step (default: decode
                     steps go first and prompts fill what is left of the token budget)
    memory_fraction  share of free device memory the page pool may take when it
                     is sized from memory
    weight_copies    keep a second copy of every matrix in the order the few-rows product streams it
                     (faster decoding at small batches, twice the memory for matrices); None decides by
                     what fits beside the cache: all, or, where they do not all fit, those that do
    weight_copy_bytes  the most bytes such copies may take (those of the matrices with the fewest rows
                     are made first); None: what is free beside the weights and the cache
    run_ahead        a step is started before the host has read the tokens of the step before it (they
                     stay on the device for it); generation is the same, tokens are reported one call later
    cast_float32_weights   bfloat16 engine: matrices stored in 32-bit are rounded to bfloat16 at load, as the
                     reference's amp='bf16' does; left False such a matrix stays in 32-bit and its product
                     runs on the float32 kernel (a line on stderr says so)
    seed             the random stream of a request whose `SamplingParams.seed` is None is keyed by this
                     plus the number of requests the engine took before it
    page_pad_bytes   device memory left between one cache page and the next (a multiple of 32; 0: none).
                     Pages of a power of two of bytes lie at distances that are powers of two, and so do
                     requests that fill them side by side; what the decode attention reads at one time then
                     falls onto the same memory channels and banks. An odd multiple of 128 bytes between pages
                     takes that regularity away (a kernel that reads as the decode attention does: 5.8 TB/s
                     at worst without, 6.2 with; OPT-6.7B, 64 requests: 16.2 -> 15.8 ms a decode step)
    """
    dtype: torch.dtype = torch.bfloat16
    page_size: int = 64
    num_pages: Optional[int] = None
    max_tokens: Optional[int] = None
    max_num_seqs: int = 64
    max_num_batched_tokens: int = 2048
    chunk_size: Optional[int] = None
    max_model_len: Optional[int] = None
    kernels: str = "hip"
    device: str = "cuda:0"
    memory_fraction: float = 0.85
    use_graphs: bool = True
    prompts_first: bool = False
    run_ahead: bool = True
    weight_copies: Optional[bool] = None
    weight_copy_bytes: Optional[int] = None
    cast_float32_weights: bool = False
    seed: int = 0
    page_pad_bytes: int = 384

    def __post_init__(self):
        self.dtype = parse_dtype(self.dtype)
        if self.page_size <= 0 or self.page_size % 16:
            raise ValueError(f"page_size must be a positive multiple of 16, got {self.page_size}")
        if self.kernels not in ("hip", "reference"):
            raise ValueError(f"kernels must be 'hip' or 'reference', got {self.kernels!r}")
        if self.max_num_seqs <= 0 or self.max_num_batched_tokens <= 0:
            raise ValueError("max_num_seqs and max_num_batched_tokens must be positive")
        if self.weight_copy_bytes is not None and self.weight_copy_bytes < 0:
            raise ValueError(f"weight_copy_bytes must not be negative, got {self.weight_copy_bytes}")
        if self.page_pad_bytes < 0 or self.page_pad_bytes % 32:
            raise ValueError(f"page_pad_bytes must be a multiple of 32 from 0 up, got {self.page_pad_bytes}")
        if self.chunk_size is not None and self.chunk_size <= 0:
            raise ValueError(f"chunk_size must be positive, got {self.chunk_size}")

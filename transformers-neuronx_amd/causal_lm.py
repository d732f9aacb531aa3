"""The user-facing model class in the reference's manner, for any registered architecture.

    model = SomeModelForSampling.from_pretrained(path, batch_size=4, amp='bf16', n_positions=2048)
    model.load()                      # `to_neuron()` is kept as another name for it
    tokens = model.sample(input_ids, sequence_length=256, top_k=50)

Reference: base.py (`NeuronModelBase`: load, save, to_neuron, forward by cache or sequence ids),
sampling.py:131-180 (the host loop behind `sample`) and module.py:395-432 (`from_pretrained`). What is
compiled and bucketed there (`tp_degree`, `unroll`, `context_length_estimate`) has no counterpart on one
GPU. An architecture's own class is this one with its `architecture` filled in.
"""
import os
import warnings
from typing import List, Optional

import torch

from .config.engine_config import EngineConfig, GenerationConfig, NeuronConfig, parse_dtype
from .config.model_config import ModelConfig
from .config.registry import Architecture, read_config
from .engine.batch import StepEntry
from .engine.engine import LLMEngine
from .engine.factory import build_runner
from .sampling.params import SamplingParams
from .weights.loader import Checkpoint


class CausalLMForSampling:
    """`tp_degree` other than 1 is refused (one GPU); `unroll`, `context_length_estimate` and `context_unroll`
    are accepted and without effect: nothing is unrolled or bucketed here."""

    architecture: Optional[Architecture] = None       # a subclass names its own; None takes any

    def __init__(self, config: ModelConfig, batch_size=1, amp=None, tp_degree=1, n_positions=2048, unroll=None,
                 context_length_estimate=None, context_unroll=1, neuron_config: Optional[NeuronConfig] = None,
                 page_size: int = 64, num_pages: Optional[int] = None, max_num_batched_tokens: int = 2048,
                 device: str = "cuda:0", kernels: str = "hip", **kwargs):
        if kwargs:
            raise KeyError(f"unknown arguments {sorted(kwargs)}")
        if tp_degree not in (1, None):
            raise ValueError(f"tp_degree={tp_degree}: this engine runs on one GPU")
        stored = getattr(config, "torch_dtype", None)
        if amp is None:
            amp = stored or "bfloat16"
        elif stored is not None and parse_dtype(amp) != parse_dtype(stored):
            warnings.warn(f"torch_dtype={stored} ignored in favor of amp={amp}")
        n_max = max(n_positions) if isinstance(n_positions, (list, tuple)) else n_positions
        from .config.registry import resolve
        self.architecture = self.architecture or resolve(config.to_dict())
        most = self.architecture.build_spec(config).max_positions
        if n_max > most:
            raise ValueError(f"Sequence length ({n_max}) cannot be larger than position embedding's context size "
                             f"({most})!")
        self.config = config
        self.neuron_config = neuron_config if neuron_config else NeuronConfig()
        self.batch_size = batch_size
        self.n_positions = n_max
        cb = self.neuron_config.continuous_batching
        max_seqs = max(batch_size if isinstance(batch_size, int) else max(batch_size),
                       cb.max_num_seqs if cb else 0)
        if cb and cb.block_size:
            page_size = cb.block_size
        if cb and cb.num_blocks:
            num_pages = cb.num_blocks
        if num_pages is None:
            num_pages = max_seqs * -(-n_max // page_size)
        self.engine_config = EngineConfig(
            dtype=parse_dtype(amp), page_size=page_size, num_pages=num_pages, max_num_seqs=max_seqs,
            max_num_batched_tokens=max_num_batched_tokens,
            max_model_len=min(n_max, cb.max_model_len) if cb and cb.max_model_len else n_max,
            device=device, kernels=kernels,
            cast_float32_weights=True)      # `amp` is the dtype of every weight, as in the reference
        self._folder: Optional[str] = None
        self._source = None
        self.engine: Optional[LLMEngine] = None

    # ---------------------------------------------------------------- construction

    @classmethod
    def from_pretrained(cls, pretrained_model_path: str, *model_args, **kwargs) -> "CausalLMForSampling":
        """Read config.json of the folder; the weights are read by `load()`."""
        arch, config = read_config(pretrained_model_path)
        if cls.architecture is not None and arch is not cls.architecture:
            raise ValueError(f"{pretrained_model_path} holds a {arch.name} model, not a {cls.architecture.name} one")
        model = cls(config, *model_args, **kwargs)
        model._folder = pretrained_model_path
        return model

    @classmethod
    def from_config(cls, config: ModelConfig, source, **kwargs) -> "CausalLMForSampling":
        """A model over tensors given in memory (`weights.TensorDict`)."""
        model = cls(config, **kwargs)
        model._source = source
        return model

    def load(self, directory: Optional[str] = None) -> "CausalLMForSampling":
        """Weights to the GPU, the page pool, the engine. (In the reference `load`
        points at precompiled artifacts, base.py:50-52, and `to_neuron` does the
        work, base.py:77-89; here both names do the one thing there is to do.)
        `directory`: a model folder to read instead of the one given at construction; a folder without a
        `config.json` is taken for the reference's folder of compiled artifacts (what `save` writes) and
        changes nothing, since nothing is compiled ahead but the kernels."""
        if directory is not None and os.path.exists(os.path.join(directory, "config.json")):
            self._folder = directory
        if self.engine is not None:
            return self
        source = self._source if self._source is not None else Checkpoint(self._folder)
        runner = build_runner(self.config, source, self.engine_config)
        self.engine = LLMEngine(runner, self.engine_config)
        return self

    def save(self, directory: str) -> None:
        """The reference stores its compiled programs here for a later `load` (base.py:39-48). The
        counterpart of compiling is building the kernels: this builds those not built yet and notes
        where they lie."""
        import json
        from .kernels import build
        os.makedirs(directory, exist_ok=True)
        with open(os.path.join(directory, "kernels.json"), "w") as fp:
            json.dump({m: build.compile_module(m) for m in build.modules()}, fp, indent=1)   # also those that parts brought

    def is_compiled(self) -> bool:
        """base.py:143-151: whether the model is ready to run."""
        return self.engine is not None

    def update_generation_config(self, generation_config: GenerationConfig) -> None:
        """base.py:761-766: other generation options from the next `sample` on."""
        self.neuron_config.on_device_generation = generation_config

    to_neuron = load

    def _need_engine(self) -> LLMEngine:
        if self.engine is None:
            raise RuntimeError("call load() (or to_neuron()) first")
        return self.engine

    # ---------------------------------------------------------------- forward, in the reference's form

    def reset(self):
        self._need_engine().reset()

    def _rows(self, input_ids, start_ids) -> List[List[int]]:
        ids = torch.as_tensor(input_ids)
        if ids.dim() == 1:
            ids = ids.unsqueeze(0)
        starts = [0] * ids.shape[0] if start_ids is None else [int(s) for s in torch.as_tensor(start_ids).flatten()]
        return [ids[b, starts[b]:].tolist() for b in range(ids.shape[0])]

    @torch.no_grad()
    def forward(self, input_ids, cache_ids=None, start_ids=None) -> torch.Tensor:
        """Logits `[batch, vocab]` of each row's last token (`[batch, tokens, vocab]` with
        `output_all_logits`, zeros where a row is padded). `cache_ids=None` starts the rows afresh with `input_ids`
        as their prompts; otherwise the tokens go on from where the rows are, and
        `cache_ids` must say so (reference: opt/model.py:158-184; rows left-padded up
        to `start_ids` lose their padding here instead of masking it)."""
        engine = self._need_engine()
        runner = engine.runner
        if self.neuron_config.continuous_batching is not None and cache_ids is not None and start_ids is not None:
            return self._forward_sequences(input_ids, cache_ids, start_ids)
        rows = self._rows(input_ids, start_ids)
        if cache_ids is None:
            # every row starts afresh, also rows of an earlier, larger batch that this one does not name
            for key in [k for k in runner.cache.requests if isinstance(k, tuple) and k[:1] == ("row",)]:
                runner.finish(key)
        else:
            first = int(torch.as_tensor(cache_ids).flatten()[0])
            for b, toks in enumerate(rows):
                have = runner.cache.num_tokens(("row", b)) if runner.cache.has(("row", b)) else 0
                shift = 0 if start_ids is None else int(torch.as_tensor(start_ids).flatten()[b])
                if first - shift != have:
                    raise ValueError(f"cache_ids start at {first}, but row {b} holds {have} tokens")
        every = self.neuron_config.output_all_logits
        entries = [StepEntry(("row", b), toks, list(range(len(toks))) if every else [len(toks) - 1])
                   for b, toks in enumerate(rows)]
        logits = runner.step(entries)
        if every:
            # `[batch, tokens, vocab]` over the width given; the places of a row's padding hold zeros
            width = max(len(toks) for toks in rows) if start_ids is None else torch.as_tensor(input_ids).shape[-1]
            out = logits.new_zeros(len(rows), width, logits.shape[-1])
            at = 0
            for b, toks in enumerate(rows):
                out[b, width - len(toks):] = logits[at:at + len(toks)]
                at += len(toks)
            return out
        return logits

    def _forward_sequences(self, input_ids, cache_ids, seq_ids) -> torch.Tensor:
        """The form a continuous-batching driver uses (base.py:500-600, :630-637): `seq_ids` (given as
        `start_ids`) name the cache rows, `cache_ids [n, tokens]` the positions the tokens take. A row
        whose positions begin at 0 starts a new sequence in that row; otherwise the tokens go on from
        where the row is. Rows not named keep what they hold. Logits come back in the order given."""
        runner = self.engine.runner
        ids = torch.as_tensor(input_ids)
        pos = torch.as_tensor(cache_ids)
        if ids.dim() == 1:
            ids = ids.unsqueeze(0)
        if pos.dim() == 1:
            pos = pos.unsqueeze(0).expand(ids.shape[0], -1)
        seqs = [int(s) for s in torch.as_tensor(seq_ids).flatten()]
        if len(seqs) != ids.shape[0] or pos.shape != ids.shape:
            raise ValueError(f"{ids.shape[0]} rows of tokens, positions of shape {tuple(pos.shape)}, {len(seqs)} seq_ids")
        every = self.neuron_config.output_all_logits
        entries = []
        for i, seq in enumerate(seqs):
            key, first = ("seq", seq), int(pos[i, 0])
            if first == 0:
                runner.finish(key)
            have = runner.cache.num_tokens(key) if runner.cache.has(key) else 0
            if first != have:
                raise ValueError(f"cache_ids start at {first}, but sequence {seq} holds {have} tokens")
            toks = ids[i].tolist()
            entries.append(StepEntry(key, toks, list(range(len(toks))) if every else [len(toks) - 1]))
        logits = runner.step(entries)
        return logits.view(len(seqs), -1, logits.shape[-1]) if every else logits

    __call__ = forward

    # ---------------------------------------------------------------- generation

    @torch.no_grad()
    def sample(self, input_ids, sequence_length: int, start_ids=None, top_k: int = 50, streamer=None,
               temperature: float = 1.0, top_p: float = 1.0, seed: int = 0,
               generation_config: Optional[GenerationConfig] = None,
               no_repeat_ngram_size: Optional[int] = None, eos_token_id: Optional[int] = None) -> torch.Tensor:
        """`[batch, sequence_length]`: the prompts and what follows them, up to a total
        length of `sequence_length`. As the reference's loop (sampling.py:131-180) it
        never picks the end-of-sequence token and keeps the `top_k` largest logits;
        `top_k=1` is greedy. With `on_device_generation` in the NeuronConfig, or a
        `generation_config`, those options decide instead (sampling.py:33-105).
        `eos_token_id`: the token the loop never picks, where it is not the configuration's.
        `no_repeat_ngram_size`: no run of that many tokens appears twice in a row's prompt and what
        follows it (the option of the reference's other loop, sampling.py:382-394)."""
        engine = self._need_engine()
        rows = self._rows(input_ids, start_ids)
        gen = generation_config or self.neuron_config.on_device_generation
        prompts = torch.as_tensor(input_ids)
        if prompts.dim() == 1:
            prompts = prompts.unsqueeze(0)
        width = prompts.shape[1]
        if sequence_length <= width:
            return prompts[:, :sequence_length].clone()
        params = []
        for b, toks in enumerate(rows):
            new = sequence_length - width
            if gen is not None:
                # config.py:106-139: values may be lists, one entry a batch line (`per_batch_line`); a global
                # top-k caps every line's own (layers/generation.py:55-56); `dynamic` needs nothing here,
                # every request carries its own options anyway
                def line(v):
                    return v[b] if isinstance(v, (list, tuple)) else v
                k = int(line(gen.top_k))
                if gen.global_top_k is not None:
                    k = min(k, int(gen.global_top_k)) if k > 0 else int(gen.global_top_k)
                p = SamplingParams(max_new_tokens=new, do_sample=gen.do_sample, temperature=float(line(gen.temperature)),
                                   top_k=k, top_p=float(line(gen.top_p)), seed=seed + b,
                                   min_tokens_to_keep=int(line(gen.top_p_min_tokens)), deterministic=gen.deterministic,
                                   eos_token_id=gen.eos_token_id, ignore_eos=gen.eos_token_id is None,
                                   no_repeat_ngram_size=int(no_repeat_ngram_size or 0))
            else:
                p = SamplingParams(max_new_tokens=new, do_sample=True, temperature=temperature, top_k=top_k,
                                   top_p=top_p, seed=seed + b,
                                   eos_token_id=(eos_token_id if eos_token_id is not None
                                                 else getattr(self.config, 'eos_token_id', None)),
                                   ban_eos=True, ignore_eos=True, no_repeat_ngram_size=int(no_repeat_ngram_size or 0))
            params.append(p)
        engine.reset()
        ids = [engine.add_request(toks, p) for toks, p in zip(rows, params)]
        column = 0              # generated tokens already handed to the streamer, the same for every row
        while engine.has_work:
            engine.step()
            if streamer is None:
                continue
            # sampling.py:159-160 hands over one token of every row at a time, `[batch, 1]`: the next column
            # goes out when every row has it or has ended (a row that ended repeats its last token's filler)
            reqs = [engine.requests[i] for i in ids]
            while column < sequence_length - width and all(
                    (len(q.output) > column and q.output[column] >= 0) or (q.finished and len(q.output) <= column)
                    for q in reqs):
                streamer.put(torch.tensor([[q.output[column] if len(q.output) > column else
                                            (p.eos_ids[0] if p.eos_ids else 0)]
                                           for q, p in zip(reqs, params)], dtype=prompts.dtype))
                column += 1
        if streamer is not None:
            streamer.end()
        result = torch.empty(len(rows), sequence_length, dtype=prompts.dtype)
        result[:, :width] = prompts
        for b, i in enumerate(ids):
            out = engine.requests[i].output
            eos = params[b].eos_ids[0] if params[b].eos_ids else 0
            out = out + [eos] * (sequence_length - width - len(out))   # rows that stopped early repeat eos
            result[b, width:] = torch.tensor(out, dtype=prompts.dtype)
        return result

"""The decoder, put together from a `ModelSpec`.

It owns the parts and their tensors and runs them in the order the spec lists.
What takes the place of the reference's graph owner
(`DecoderLmHeadForSamplingNoEmbedding`, decoder.py:43-1115, with its 26 named
weight slots per layer, :1275-1312) is this loop over parts that launch kernels.
"""
from typing import Dict, List, Optional

import torch

from ..parts.base import BLOCKS, EMBEDDINGS, FEED_FORWARDS, HEADS, MIXERS, NORMS, CacheNeed, Stream
from ..parts.spec import LayerSpec, ModelSpec, ParamDecl
from ..weights.loader import load_tensors
from .. import debug


class _Layer:
    def __init__(self, spec: LayerSpec):
        self.spec = spec
        self.mixer = MIXERS.build(spec.mixer)
        self.feed_forward = FEED_FORWARDS.build(spec.feed_forward)
        self.mixer_norm = NORMS.build(spec.mixer_norm)
        self.feed_forward_norm = NORMS.build(spec.feed_forward_norm)
        self.block = BLOCKS.build(
            _spec_of(spec.block), self.mixer, self.feed_forward, self.mixer_norm, self.feed_forward_norm)

    def _named(self):
        s = self.spec
        return [(self.mixer, s.prefix + s.mixer_name), (self.feed_forward, s.prefix + s.feed_forward_name),
                (self.mixer_norm, s.prefix + s.mixer_norm_name),
                (self.feed_forward_norm, s.prefix + s.feed_forward_norm_name)]

    def param_decls(self) -> List[ParamDecl]:
        return [d for part, prefix in self._named() for d in part.param_decls(prefix)]

    def load(self, tensors, ops, dtype, finish=True):
        for part, prefix in self._named():
            part.load(tensors, prefix, ops, dtype)
        if finish:
            self.block.after_load()


def _spec_of(kind):
    from ..parts.spec import PartSpec
    return kind if isinstance(kind, PartSpec) else PartSpec(kind)


class DecoderModel:
    def __init__(self, spec: ModelSpec):
        self.spec = spec
        self.embedding = EMBEDDINGS.build(spec.embedding)
        self.layers = [_Layer(ls) for ls in spec.layers]
        self.head = HEADS.build(spec.head)
        self.schedule = spec.resolved_schedule()
        written = set()
        for layer, cid, writes in self.schedule:
            if writes:
                written.add(cid)
            elif cid not in written:
                raise ValueError(f"layer {layer} reads cache {cid} before the call that writes it")
        self.loaded = False
        parts = [self.embedding, self.embedding.position, self.head] + ([self.head.norm] if self.head.norm else [])
        for l in self.layers:
            parts += [l.block, l.mixer, l.feed_forward, l.mixer_norm, l.feed_forward_norm]
        self.recordable = all(getattr(p, "recordable", False) for p in parts)
        self.parts = [p for p in parts if p is not None]

    # ---------------------------------------------------------------- declarations

    def param_decls(self) -> List[ParamDecl]:
        decls, seen = [], set()
        for d in (self.embedding.param_decls() + [d for l in self.layers for d in l.param_decls()]
                  + self.head.param_decls()):
            if d.name not in seen:
                seen.add(d.name)
                decls.append(d)
        return decls

    def cache_needs(self) -> Dict[int, Optional[CacheNeed]]:
        """{cache id: need} of the calls that write a cache."""
        return {cid: self.layers[layer].mixer.cache_need() for layer, cid, writes in self.schedule if writes}

    def step_planners(self) -> Dict[str, object]:
        """The step planners that the parts bring with them."""
        out: Dict[str, object] = {}
        for part in self.parts:
            out.update(part.step_planners())
        return out

    def launch_shape(self, step) -> tuple:
        """What the parts' launches of a decode step are sized by, beyond its layout (`Part.launch_shape`)."""
        shapes = []
        for part in self.parts:
            shape = part.launch_shape(step)
            if shape is not None and shape not in shapes:
                shapes.append(shape)
        return tuple(shapes)

    # ---------------------------------------------------------------- accounting (for measurements)

    def step_flops(self, tokens: float, keys: float, wanted: float) -> float:
        """Multiply-adds times two of a step of `tokens` tokens that see `keys` cached tokens each on
        average (a whole prompt of T tokens: (T + 1) / 2) and ask for `wanted` rows of logits."""
        per_token = self.embedding.flops_per_token(keys)
        for layer, _, _ in self.schedule:
            l = self.layers[layer]
            per_token += sum(p.flops_per_token(keys) for p in (l.mixer, l.feed_forward, l.mixer_norm, l.feed_forward_norm))
        return tokens * per_token + wanted * self.head.flops_per_token(keys)

    def cache_bytes_read(self, keys: float, dtype: torch.dtype, page_size: int = 1) -> float:
        """Bytes of its request's cache that one decoded token reads at a context of `keys` tokens: every call
        of the run order reads the cache it names (a windowed one up to its window)."""
        needs = {cid: self.layers[layer].mixer.cache_need() for layer, cid, writes in self.schedule if writes}
        total = 0.0
        for _, cid, _ in self.schedule:
            need = needs.get(cid)
            if need is None or need.kind != "paged":
                continue
            from ..cache.manager import CacheManager
            per_token = CacheManager.bytes_per_page({0: need}, page_size, dtype) / page_size
            total += per_token * (min(keys, need.window) if need.window else keys)
        return total

    # ---------------------------------------------------------------- weights

    def load(self, source, ops, dtype: torch.dtype, device, cast_float32: bool = False,
             finish: bool = True) -> "DecoderModel":
        """`finish=False` leaves out what the blocks do once their parts have their tensors (`finish_load`
        does it later: the caller has something to do to the weights in between)."""
        tensors = load_tensors(self.param_decls(), source, dtype, device, self.spec.base_model_prefix, cast_float32)
        self.embedding.load(tensors, "", ops, dtype)
        for layer in self.layers:
            layer.load(tensors, ops, dtype, finish)
        self.head.load(tensors, "", ops, dtype)
        self.ops, self.dtype, self.device = ops, dtype, device
        self.weight_bytes = sum(t.numel() * t.element_size() for t in {id(t): t for t in tensors.values()}.values())
        self.loaded = True
        return self

    def finish_load(self) -> None:
        for layer in self.layers:
            layer.block.after_load()

    # ---------------------------------------------------------------- one step

    def forward(self, ctx, caches) -> torch.Tensor:
        """Logits float32 `[len(ctx.logits_rows), vocab]` for the step `ctx` describes."""
        first_block = self.layers[self.schedule[0][0]].block if self.schedule else None
        want_compute = bool(getattr(first_block, "reads_compute_copy", False))
        stream: Stream = self.embedding.forward(ctx, want_compute)
        debug.tap("embedding", stream.x)
        for call, (layer, cid, writes) in enumerate(self.schedule):
            cache = caches[cid] if writes else caches[cid].reader()
            stream = self.layers[layer].block.forward(stream, ctx, cache)
            debug.tap(f"call{call}.layer{layer}", stream.x)
        return debug.tap("logits", self.head.forward(stream, ctx))


def model_param_decls(spec: ModelSpec) -> List[ParamDecl]:
    return DecoderModel(spec).param_decls()

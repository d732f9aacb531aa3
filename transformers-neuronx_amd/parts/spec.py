"""The description of a model as data: which parts make up each layer, with which
sizes and constants, and in which order the layers run.

An architecture is a function from its typed configuration to a `ModelSpec`;
the model builder, the weight loader, the cache manager and the step function
read the spec and nothing else. No part knows which model it is in.
"""
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Tuple


@dataclass(frozen=True)
class PartSpec:
    """One part: the name it is registered under and its parameters."""
    kind: str
    params: Dict[str, Any] = field(default_factory=dict)

    def __hash__(self):
        return hash((self.kind, tuple(sorted((k, repr(v)) for k, v in self.params.items()))))


@dataclass(frozen=True)
class ParamDecl:
    """A tensor a part reads from the checkpoint.

    role    'matrix' (operand of a matrix product, kept in the compute dtype),
            'table' (rows are looked up, kept in the compute dtype),
            'vector' (bias or norm parameter, kept in float32),
            'index' (integer table, kept in int32)
    init    how the random-weights mode draws it: 'normal' (mean 0),
            'around_one' (mean 1), both with the configuration's deviation
    tied_to another tensor's name that stands in when this one is absent
    """
    name: str
    shape: Tuple[int, ...]
    role: str = "matrix"
    init: str = "normal"
    tied_to: Optional[str] = None


@dataclass(frozen=True)
class LayerSpec:
    """One layer: a block arrangement and the four parts it arranges.

    `prefix` is the checkpoint name prefix of the layer; each part's parameter
    names are relative to it (the `*_name` fields)."""
    prefix: str
    block: str                      # registered arrangement, e.g. "pre_norm"
    mixer: PartSpec
    feed_forward: PartSpec
    mixer_norm: PartSpec
    feed_forward_norm: PartSpec
    mixer_name: str = "mixer"
    feed_forward_name: str = ""
    mixer_norm_name: str = "mixer_norm"
    feed_forward_norm_name: str = "feed_forward_norm"


@dataclass(frozen=True)
class LayerCall:
    """One entry of the run order.

    layer   index into `ModelSpec.layers` (a layer may be named more than once:
            its weights are shared)
    cache   id of the cache this call uses; calls with the same id share one
            cache. None means a cache of its own.
    writes  whether this call stores into that cache; a call that only reads
            another call's cache has writes=False
    """
    layer: int
    cache: Optional[int] = None
    writes: bool = True


@dataclass(frozen=True)
class ModelSpec:
    hidden_size: int
    vocab_size: int
    max_positions: int
    embedding: PartSpec             # token table, optional projection, position encoding at the input
    layers: Tuple[LayerSpec, ...]
    schedule: Tuple[LayerCall, ...]
    head: PartSpec                  # final norm, optional projection, vocabulary projection
    init_std: float = 0.02
    # A checkpoint of the base model alone names its tensors without this leading piece; the loader
    # tries a declared name without it when the name itself is absent ("" : no such form).
    base_model_prefix: str = ""

    @staticmethod
    def sequential(n_layers: int) -> Tuple[LayerCall, ...]:
        return tuple(LayerCall(i) for i in range(n_layers))

    def resolved_schedule(self) -> List[Tuple[int, int, bool]]:
        """(layer, cache id, writes) with own caches numbered after the given ids."""
        given = [c.cache for c in self.schedule if c.cache is not None]
        nxt = (max(given) + 1) if given else 0
        out = []
        for call in self.schedule:
            if not 0 <= call.layer < len(self.layers):
                raise ValueError(f"run order names layer {call.layer}; the model has {len(self.layers)}")
            cid = call.cache
            if cid is None:
                cid = nxt
                nxt += 1
            out.append((call.layer, cid, call.writes))
        writers = {}
        for layer, cid, writes in out:
            if writes:
                if cid in writers:
                    raise ValueError(f"cache {cid} is written by two calls of the run order")
                writers[cid] = layer
        for layer, cid, writes in out:
            if not writes and cid not in writers:
                raise ValueError(f"a call reads cache {cid}, which no call writes")
        return out

"""Interfaces of the parts and the registries they are found in.

A part is built from the parameters of its `PartSpec`, declares the tensors it
reads (`param_decls`), receives them (`load`) and is called by a block with the
step's context. Mixers also declare what they keep between steps
(`cache_need`). Registering a class under a new kind is all it takes to use it
from a `ModelSpec`.
"""
from dataclasses import dataclass
from typing import Callable, Dict, Hashable, List, Optional, Tuple

from .spec import ParamDecl, PartSpec


@dataclass(frozen=True)
class CacheNeed:
    """What a mixer keeps per request between steps.

    kind 'paged': grows with the tokens, in pages. What a page holds is a set of named tensors,
         `page_tensors` = ((name, shape), ...), where the place of the page's tokens in a shape is the
         string "page" (the manager puts its page size there and the page number in front). Left empty,
         it is what attention keeps: keys `(kv_heads, "page", head_size)` and values
         `(kv_heads, head_size, "page")`. `window` (tokens) lets pages be given back once every later
         query is past them, None keeps them all.
    kind 'state': fixed size per request. `state_shapes` is ((name, dims), ...); a slot is zeroed when a
         request gets it.
    """
    kind: str
    kv_heads: int = 0
    head_size: int = 0
    window: Optional[int] = None
    state_shapes: Tuple[Tuple[str, Tuple[int, ...]], ...] = ()
    state_dtype: str = "float32"
    page_tensors: Tuple[Tuple[str, Tuple], ...] = ()

    def group_key(self):
        """Layers with equal keys share a page table."""
        return (self.kind, self.window)

    def tensors_of_a_page(self) -> Tuple[Tuple[str, Tuple], ...]:
        if self.page_tensors:
            return self.page_tensors
        return (("k", (self.kv_heads, "page", self.head_size)), ("v", (self.kv_heads, self.head_size, "page")))


class Part:
    """Base of all parts. `ops` is the kernel backend, `dtype` the compute dtype.

    `recordable` says that a step through this part may be recorded once and replayed: everything it
    does is a launch on the current stream whose sizes depend on the number of tokens and requests
    only, and it reads nothing of the step on the host. Parts that loop over requests in Python, or
    index tensors with host values of the step, leave it False; a model with such a part is never
    recorded."""

    recordable = False

    def param_decls(self, prefix: str) -> List[ParamDecl]:
        return []

    def load(self, tensors: Dict[str, "object"], prefix: str, ops, dtype) -> None:
        self.ops = ops
        self.dtype = dtype

    def step_planners(self) -> Dict[str, Callable]:
        """{name: planner} of what this part's kernels want laid out with every step's integers
        (`engine.batch`): `fn(run_lens, cached, page_size) -> ({name: int32 array}, {name: host value})`."""
        return {}

    def launch_shape(self, step) -> Optional[Hashable]:
        """What this part's launches in a decode step are sized by beyond the number of requests, for a
        `PackedStep` about to be replayed from a recording: two steps share a recording only where every
        part gives the same answer. None: nothing."""
        return None

    def flops_per_token(self, keys: float = 0.0) -> float:
        """Multiply-adds times two that one token costs in this part, for a measurement's accounting; `keys`
        is the number of cached tokens of its request that the token sees. By default every declared
        matrix meets every token once; a part that does otherwise (experts of which a token takes some,
        products over the cache) says so."""
        count = 0
        for d in self.param_decls(""):
            if d.role == "matrix":
                n = 1
                for dim in d.shape:
                    n *= dim
                count += n
        return 2.0 * count


class Mixer(Part):
    """Mixes information between the tokens of a request.

    forward(h, ctx, cache, residual) -> float32 `[T, hidden]`: residual + mix(h).
    `h` is `[T, hidden]` in the compute dtype, `cache` the `LayerCache` of the
    call (None if `cache_need()` is None), `ctx` the step's `StepContext`. The
    result must not depend on how a request's tokens were cut into steps.
    """

    def cache_need(self) -> Optional[CacheNeed]:
        return None

    def forward(self, h, ctx, cache, residual):
        raise NotImplementedError

    def first_weight(self):
        """The matrix that `h` is multiplied by, if that product is all this part does with `h` and it goes
        through `ops.linear` or `ops.qkv_project`; None otherwise. A block may then hand `h` over as
        what `Norm.deferred` returns and let the product apply the norm."""
        return None


class FeedForward(Part):
    """forward(h, ctx, residual) -> float32 `[T, hidden]`: residual + f(h), token by token."""

    def forward(self, h, ctx, residual):
        raise NotImplementedError

    def first_weight(self):
        """As `Mixer.first_weight`."""
        return None


class Norm(Part):
    """forward(x, want_f32, want_compute) -> (float32 or None, compute dtype or None),
    both `[T, hidden]`, from the float32 `x`. Statistics are taken in float32."""

    def forward(self, x, want_f32: bool, want_compute: bool):
        raise NotImplementedError

    def fold_into(self, w) -> bool:
        """Asked once, after loading, by a block whose next part only multiplies this norm's output by `w`:
        True if the backend has folded the norm into `w`, so that `deferred` may be used for that part."""
        return False

    def deferred(self, x):
        """The compute-dtype output for a part whose `first_weight` this norm was folded into: the output
        itself, or what the backend's products take in its place."""
        return self.forward(x, False, True)[1]


class PositionEncoding(Part):
    """Where positions enter. `at_input(x, positions, want_compute)` adds to the embedded tokens (learned or
    fixed tables) and returns `(float32, compute dtype or None)`. `on_query_key(qkv, ctx, num_heads,
    num_kv_heads, head_size)` is the hook of encodings that turn queries and keys inside a mixer: the
    attention mixer calls it, when its spec names such an encoding as `rotation`, with the step's
    `[T, (num_heads + 2 num_kv_heads) * head_size]` projections (bias added, query not yet scaled) and
    `ctx.positions`, and stores what it returns; or, for the common pairwise form, with nothing at all:
    see `pair_tables`. A part leaves the hook it does not use as it is."""

    def at_input(self, x, positions, want_compute: bool):
        return None

    def on_query_key(self, qkv, ctx, num_heads: int, num_kv_heads: int, head_size: int):
        return qkv

    def pair_tables(self, head_size: int):
        """For an encoding that turns queries and keys pair by pair: float32 tables `(a, b)`, both
        `[positions, head_size]`, such that element d of a head of the token at position p becomes
        a[p, d] x[d] + b[p, d] x[d ^ 1]; asked once, after loading. The attention mixer then hands them to the
        projection, which applies them where it adds the bias, in the same launch, and `on_query_key` is not
        called; such a part may be `recordable`. None (the default): the encoding is not of that form. An
        encoding that pairs element d with d + head_size / 2 is of that form once the rows of the query and
        key projections are put in the order (0, h/2, 1, h/2 + 1, ...) in every head, which changes no score."""
        return None


class Block(Part):
    """Arranges one layer's mixer, feed-forward and norms around the residual stream.

    forward(stream, ctx, cache) -> stream, where stream is a `Stream`."""

    def __init__(self, mixer: Mixer, feed_forward: FeedForward, mixer_norm: Norm, feed_forward_norm: Norm):
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.mixer_norm = mixer_norm
        self.feed_forward_norm = feed_forward_norm

    def after_load(self) -> None:
        """Called when the four parts have their tensors."""

    def forward(self, stream, ctx, cache):
        raise NotImplementedError


@dataclass
class Stream:
    """The residual stream between layers: float32 `[T, hidden]`, and beside it a
    copy in the compute dtype when the last part that wrote it made one."""
    x: "object"
    compute: Optional["object"] = None


class _Registry:
    def __init__(self, what: str):
        self.what = what
        self._classes: Dict[str, type] = {}

    def register(self, kind: str) -> Callable[[type], type]:
        def deco(cls):
            self._classes[kind] = cls
            cls.kind = kind
            return cls
        return deco

    def build(self, spec: PartSpec, *args):
        if spec.kind not in self._classes:
            raise KeyError(f"no {self.what} is registered as {spec.kind!r}; known: {sorted(self._classes)}")
        return self._classes[spec.kind](*args, **spec.params)

    def kinds(self):
        return sorted(self._classes)


MIXERS = _Registry("mixer")
FEED_FORWARDS = _Registry("feed-forward")
NORMS = _Registry("norm")
POSITIONS = _Registry("position encoding")
BLOCKS = _Registry("block arrangement")
EMBEDDINGS = _Registry("embedding")
HEADS = _Registry("head")

register_mixer = MIXERS.register
register_feed_forward = FEED_FORWARDS.register
register_norm = NORMS.register
register_position = POSITIONS.register
register_block = BLOCKS.register
register_embedding = EMBEDDINGS.register
register_head = HEADS.register

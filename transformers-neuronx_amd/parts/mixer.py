"""Token mixers."""
import math
from typing import Dict, List, Optional

import torch

from .base import POSITIONS, CacheNeed, Mixer, register_mixer
from .spec import ParamDecl


@register_mixer("attention")
class Attention(Mixer):
    """Softmax attention over a paged key/value cache.

    `Q = (h Wq^T + bq) * scale`, keys and values of the step's tokens are stored
    into the request's pages, each query attends to the keys of its own request
    at positions `<=` its own (and `> position - window` when a window is set),
    softmax in float32, then the output projection (reference:
    opt/model.py:444-523; scale layers/attention.py:428-437; masks
    hlo.py:1030-1042 and the bottom-right block-diagonal form hlo.py:3211-3309;
    cache scatter by slot hlo.py:3665-3704).

    `num_kv_heads < num_heads` groups query heads over shared key/value heads.
    `own_kv=False` builds a mixer without key/value projections that reads the
    cache another call of the run order writes. `rotation` names a position
    encoding (a `PartSpec` of the position registry) that turns the queries and
    keys before they are scaled and stored: through its `pair_tables`, inside the
    projection's launch, or else through its `on_query_key`; OPT has none.
    """

    recordable = True

    def __init__(self, width: int, num_heads: int, head_size: int, names, num_kv_heads: Optional[int] = None,
                 bias: bool = True, window: Optional[int] = None, scale: Optional[float] = None,
                 own_kv: bool = True, rotation=None):
        """`names`: the checkpoint's names of the query, key, value and output projections, relative to
        the mixer's prefix (the architecture's spec gives them)."""
        self.width, self.num_heads, self.head_size = width, num_heads, head_size
        self.num_kv_heads = num_kv_heads if num_kv_heads is not None else num_heads
        if self.num_heads % self.num_kv_heads:
            raise ValueError(f"num_heads ({num_heads}) must be a multiple of num_kv_heads ({self.num_kv_heads})")
        if head_size % 16 or not 16 <= head_size <= 256:
            raise ValueError(f"head_size must be a multiple of 16 between 16 and 256, got {head_size}")
        self.has_bias, self.window, self.own_kv = bias, window, own_kv
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(head_size)
        self.names = tuple(names)
        self.rotation = POSITIONS.build(rotation) if rotation is not None else None
        if self.rotation is not None and not getattr(self.rotation, "recordable", False):
            self.recordable = False
        if len(self.names) != 4:
            raise ValueError("names: the query, key, value and output projections, four names")

    def cache_need(self) -> Optional[CacheNeed]:
        return CacheNeed("paged", kv_heads=self.num_kv_heads, head_size=self.head_size, window=self.window)

    def param_decls(self, prefix: str) -> List[ParamDecl]:
        qn, kn, vn, on = self.names
        q_out = self.num_heads * self.head_size
        kv_out = self.num_kv_heads * self.head_size
        outs = [(qn, q_out)] + ([(kn, kv_out), (vn, kv_out)] if self.own_kv else [])
        d = []
        for n, out in outs:
            d.append(ParamDecl(f"{prefix}{n}.weight", (out, self.width)))
            if self.has_bias:
                d.append(ParamDecl(f"{prefix}{n}.bias", (out,), "vector"))
        d.append(ParamDecl(f"{prefix}{on}.weight", (self.width, q_out)))
        if self.has_bias:
            d.append(ParamDecl(f"{prefix}{on}.bias", (self.width,), "vector"))
        if self.rotation is not None:
            d += self.rotation.param_decls(prefix + "rotation")
        return d

    def load(self, tensors: Dict, prefix: str, ops, dtype) -> None:
        super().load(tensors, prefix, ops, dtype)
        qn, kn, vn, on = self.names
        ins = [qn] + ([kn, vn] if self.own_kv else [])
        # One fused projection: a plain concatenation of the rows (the reference's
        # fused form interleaves per tensor-parallel shard, utils.py:189-242).
        self.w_qkv = ops.prepare_weight(torch.cat([tensors[f"{prefix}{n}.weight"] for n in ins], dim=0).contiguous())
        self.b_qkv = (torch.cat([tensors[f"{prefix}{n}.bias"] for n in ins], dim=0).contiguous()
                      if self.has_bias else None)
        self.w_out = ops.prepare_weight(tensors[f"{prefix}{on}.weight"])
        self.b_out = tensors[f"{prefix}{on}.bias"] if self.has_bias else None
        self.turn = None
        if self.rotation is not None:
            self.rotation.load(tensors, prefix + "rotation", ops, dtype)
            self.turn = self.rotation.pair_tables(self.head_size)     # the pairwise form: applied by the projection

    def first_weight(self):
        return self.w_qkv

    def step_planners(self):
        from ..kernels.attention_plan import attention_plan
        return {"attention": attention_plan}

    def launch_shape(self, step):
        shape = getattr(self.ops, "attention_launch_shape", None)
        return shape(step, self.num_heads, self.window, self.head_size, self.num_kv_heads) if shape is not None else None

    def flops_per_token(self, keys: float = 0.0) -> float:
        seen = min(keys, self.window) if self.window else keys
        return super().flops_per_token(keys) + 4.0 * self.num_heads * self.head_size * seen   # q k^T and p v

    def forward(self, h, ctx, cache, residual):
        if cache.writes != self.own_kv:
            raise ValueError("an attention mixer with own_kv writes its cache; one without reads another's")
        view = ctx.groups[cache.group]
        kv_write = self.num_kv_heads if self.own_kv else 0
        if self.rotation is not None and self.turn is None:
            # the projections with their bias, turned by the encoding, then scaled and stored
            qkv = self.ops.linear(h, self.w_qkv, self.b_qkv)
            qkv = self.rotation.on_query_key(qkv, ctx, self.num_heads, kv_write, self.head_size)
            q = self.ops.qkv_write(qkv, None, self.num_heads, kv_write, self.head_size, self.scale, ctx, view,
                                   cache.k_pages, cache.v_pages)
            c = self.ops.attention(q, self.num_heads, self.num_kv_heads, self.head_size, ctx, view,
                                   cache.k_pages, cache.v_pages, self.window)
            return self.ops.linear(c, self.w_out, self.b_out, residual=residual, out_f32=True)
        q = self.ops.qkv_project(h, self.w_qkv, self.b_qkv, self.num_heads,
                                 self.num_kv_heads if self.own_kv else 0, self.head_size, self.scale, ctx, view,
                                 cache.k_pages, cache.v_pages, **({"turn": self.turn} if self.turn is not None else {}))
        c = self.ops.attention(q, self.num_heads, self.num_kv_heads, self.head_size, ctx, view,
                               cache.k_pages, cache.v_pages, self.window)
        return self.ops.linear(c, self.w_out, self.b_out, residual=residual, out_f32=True)

"""Feed-forward parts."""
from typing import Dict, List

from .base import FeedForward, register_feed_forward
from .spec import ParamDecl


@register_feed_forward("dense")
class DenseFeedForward(FeedForward):
    """`act(h W1^T + b1) W2^T + b2`, the activation applied to the float32
    accumulator (reference: hlo.py:550-559; activations.py:20-48)."""

    recordable = True

    def __init__(self, width: int, inner: int, activation: str, up_name: str, down_name: str, bias: bool = True):
        """`up_name`, `down_name`: the checkpoint's names of the two matrices, relative to the part's prefix."""
        self.width, self.inner, self.activation, self.has_bias = width, inner, activation, bias
        self.up_name, self.down_name = up_name, down_name

    def param_decls(self, prefix: str) -> List[ParamDecl]:
        d = [ParamDecl(f"{prefix}{self.up_name}.weight", (self.inner, self.width)),
             ParamDecl(f"{prefix}{self.down_name}.weight", (self.width, self.inner))]
        if self.has_bias:
            d += [ParamDecl(f"{prefix}{self.up_name}.bias", (self.inner,), "vector"),
                  ParamDecl(f"{prefix}{self.down_name}.bias", (self.width,), "vector")]
        return d

    def load(self, tensors: Dict, prefix: str, ops, dtype) -> None:
        super().load(tensors, prefix, ops, dtype)
        self.w1 = ops.prepare_weight(tensors[f"{prefix}{self.up_name}.weight"])
        self.w2 = ops.prepare_weight(tensors[f"{prefix}{self.down_name}.weight"])
        self.b1 = tensors.get(f"{prefix}{self.up_name}.bias") if self.has_bias else None
        self.b2 = tensors.get(f"{prefix}{self.down_name}.bias") if self.has_bias else None

    def first_weight(self):
        return self.w1

    def forward(self, h, ctx, residual):
        inner = self.ops.linear(h, self.w1, self.b1, act=self.activation)
        return self.ops.linear(inner, self.w2, self.b2, residual=residual, out_f32=True)

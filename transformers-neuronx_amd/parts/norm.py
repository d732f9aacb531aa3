"""Norm parts."""
from typing import Dict, List

from .base import Norm, register_norm
from .spec import ParamDecl


@register_norm("layer_norm")
class LayerNorm(Norm):
    """Mean and biased variance over the width in float32, `(x - mean) *
    rsqrt(var + eps)`, then weight and bias when `affine`
    (reference: hlo.py:84-105, eps of hlo.py:51 passed in as a parameter)."""

    recordable = True

    def __init__(self, width: int, eps: float, affine: bool = True):
        self.width, self.eps, self.affine = width, float(eps), affine
        self.weight = self.bias = None

    def param_decls(self, prefix: str) -> List[ParamDecl]:
        if not self.affine:
            return []
        return [ParamDecl(prefix + ".weight", (self.width,), "vector", "around_one"),
                ParamDecl(prefix + ".bias", (self.width,), "vector", "normal")]

    def load(self, tensors: Dict, prefix: str, ops, dtype) -> None:
        super().load(tensors, prefix, ops, dtype)
        if self.affine:
            self.weight = tensors[prefix + ".weight"]
            self.bias = tensors[prefix + ".bias"]

    def forward(self, x, want_f32: bool, want_compute: bool):
        return self.ops.layernorm(x, self.weight, self.bias, self.eps, self.dtype, want_f32, want_compute)

    def fold_into(self, w) -> bool:
        return self.ops.fold_norm(w, self.weight, self.bias)

    def deferred(self, x):
        return self.ops.layernorm_deferred(x, self.weight, self.bias, self.eps, self.dtype)

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

    def __init__(self, width: int, eps: float, affine: bool = True, weight_suffix: str = ".weight",
                 bias_suffix: str = ".bias", bias: bool = True):
        """`weight_suffix`, `bias_suffix`: what the checkpoint's names of the two vectors add to the norm's;
        `bias=False`: an affine norm with a weight alone."""
        self.width, self.eps, self.affine = width, float(eps), affine
        self.has_bias = bool(bias) and affine
        self.weight_suffix, self.bias_suffix = weight_suffix, bias_suffix
        self.weight = self.bias = None

    def param_decls(self, prefix: str) -> List[ParamDecl]:
        if not self.affine:
            return []
        d = [ParamDecl(prefix + self.weight_suffix, (self.width,), "vector", "around_one")]
        if self.has_bias:
            d.append(ParamDecl(prefix + self.bias_suffix, (self.width,), "vector", "normal"))
        return d

    def load(self, tensors: Dict, prefix: str, ops, dtype) -> None:
        super().load(tensors, prefix, ops, dtype)
        if self.affine:
            self.weight = tensors[prefix + self.weight_suffix]
            self.bias = tensors[prefix + self.bias_suffix] if self.has_bias else None

    def forward(self, x, want_f32: bool, want_compute: bool):
        return self.ops.layernorm(x, self.weight, self.bias, self.eps, self.dtype, want_f32, want_compute)

    def add_to(self, y, residual, mult: float = 1.0, out=None, want_compute: bool = False):
        """`residual + mult * norm(y)` in float32 (into `out`, if given): the norm that follows a part."""
        return self.ops.norm_add(y, self.weight, self.bias, self.eps, True, residual, mult, out, want_compute)

    def fused_form(self):
        """(weight, bias, center, eps) for kernels that apply the norm inside a launch of their own."""
        return self.weight, self.bias, True, self.eps

    def fold_into(self, w) -> bool:
        return self.ops.fold_norm(w, self.weight, self.bias)

    def deferred(self, x):
        return self.ops.layernorm_deferred(x, self.weight, self.bias, self.eps, self.dtype)


@register_norm("rms_norm")
class RMSNorm(Norm):
    """`x / sqrt(mean(x^2) + eps) * weight`, statistics in float32: the norm that only scales. With `unit_offset`
    the checkpoint stores the weight around zero and the factor is `1 + weight` (the sum is made once, at load,
    in float32)."""

    recordable = True

    def __init__(self, width: int, eps: float, weight_suffix: str = ".weight", unit_offset: bool = False,
                 scalar: bool = False):
        """`scalar`: the checkpoint's weight is one number (a tensor without dimensions) that multiplies every
        coordinate; it is spread over the width once, at load."""
        self.width, self.eps, self.weight_suffix = width, float(eps), weight_suffix
        self.unit_offset, self.scalar = bool(unit_offset), bool(scalar)
        self.weight = None

    def param_decls(self, prefix: str) -> List[ParamDecl]:
        return [ParamDecl(prefix + self.weight_suffix, () if self.scalar else (self.width,), "vector",
                          "normal" if self.unit_offset else "around_one")]

    def load(self, tensors: Dict, prefix: str, ops, dtype) -> None:
        super().load(tensors, prefix, ops, dtype)
        self.weight = tensors[prefix + self.weight_suffix]
        if self.scalar:
            self.weight = self.weight.reshape(1).expand(self.width).contiguous()
        if self.unit_offset:
            self.weight = (self.weight.float() + 1.0).contiguous()

    def forward(self, x, want_f32: bool, want_compute: bool):
        return self.ops.layernorm(x, self.weight, None, self.eps, self.dtype, want_f32, want_compute, center=False)

    def add_to(self, y, residual, mult: float = 1.0, out=None, want_compute: bool = False):
        return self.ops.norm_add(y, self.weight, None, self.eps, False, residual, mult, out, want_compute)

    def fused_form(self):
        return self.weight, None, False, self.eps

    def fold_into(self, w) -> bool:
        return self.ops.fold_norm(w, self.weight, None, center=False)

    def deferred(self, x):
        return self.ops.layernorm_deferred(x, self.weight, None, self.eps, self.dtype, center=False)

"""Norm parts.  Interface of a norm:

    params(spec) -> {local name: ParamSpec}
    load(tensors)                       tensors by local name, already on the device
    forward(x, out_dtype) -> y          x float32 [rows, width]
    add_forward(x, delta, out_dtype)    x += delta in place, then y = norm(x)
    post_forward(x, delta, alpha, rows_dtype) -> rows
                                        x = norm(alpha x + delta) in place (the norm after the sum, whose result IS
                                        the residual stream); `rows`: the same in `rows_dtype` for the next products
                                        (x itself where that is float32).  Optional: what a post-norm block needs.

A norm with `fuses_products = True` also takes a delta that `Runtime.linear(...,
defer=True)` has not launched yet and may return `ScaledRows` (its rows without
their scale, which the product that follows applies); blocks settle both for
parts that do not say they take them.
"""
from __future__ import annotations

from ..runtime import Deferred, Pending, WeightedDelta
from .base import ParamSpec, register


@register("norm", "rms_norm")
class RMSNorm:
    """y = x * rsqrt(mean(x^2) + eps) * w  (/root/reference/src/kipp.c:2221-2231)."""

    graph_safe = True   # forward launches kernels only: no host reads, no data-dependent launches
    fuses_products = True

    def __init__(self, spec, runtime):
        self.spec = spec
        self.rt = runtime
        self.weight = None

    @staticmethod
    def params(spec):
        return {getattr(spec, "name", "weight"): ParamSpec((spec.width,), "float", ("one_plus_normal", 0.05))}

    @staticmethod
    def placement(spec):
        """Norm weights are widened to float32 on the device (exact)."""
        return {getattr(spec, "name", "weight"): "float32"}

    def load(self, tensors):
        self.weight = tensors[getattr(self.spec, "name", "weight")]

    def forward(self, x, out_dtype):
        return self.rt.ops.rmsnorm(x, self.weight, self.spec.eps, self.rt.empty(x.shape, out_dtype))

    def add_forward(self, x, delta, out_dtype):
        if isinstance(delta, Deferred):       # a product not launched yet: add and norm ride on it where they can
            fused = self.rt.product_add_norm(delta, x, self.weight, self.spec.eps) if out_dtype == self.rt.act_dtype else None
            if fused is not None:
                return fused
            delta = delta.run()
        elif isinstance(delta, WeightedDelta):
            delta.add_to(x)         # every term where it lies, then the norm alone
            return self.forward(x, out_dtype)
        elif isinstance(delta, Pending):
            delta = delta.run()
        return self.rt.ops.rmsnorm(x, self.weight, self.spec.eps, self.rt.empty(x.shape, out_dtype), delta=delta)

    def post_forward(self, x, delta, alpha, rows_dtype):
        import torch
        delta = self.rt.settle(delta)
        rows = None if rows_dtype == torch.float32 else self.rt.empty(x.shape, rows_dtype)
        self.rt.ops.scaled_add_rmsnorm(x, delta, alpha, self.weight, self.spec.eps, rows)
        return x if rows is None else rows


@register("norm", "rms_norm_one_plus")
class OnePlusRMSNorm(RMSNorm):
    """y = x * rsqrt(mean(x^2) + eps) * (1 + w): the tensor holds the offset of the weight from one.  The one is added once, at
    load, in float32; from there on it is the plain norm and rides on the same kernels."""

    @staticmethod
    def params(spec):
        return {spec.name: ParamSpec((spec.width,), "float", ("normal", 0.05))}

    @staticmethod
    def placement(spec):
        return {spec.name: "float32"}

    def load(self, tensors):
        self.weight = (tensors[self.spec.name].float() + 1.0).contiguous()


class NormedDelta(Pending):
    """A sublayer's result that is still to be normed, scaled and added: x += mult * norm(delta) [+ extra].  The norm in front
    of the next sublayer (`LayerNorm.add_forward`) carries it out in its own kernel; `run()` gives the addend as a tensor."""
    __slots__ = ("rt", "delta", "norm", "mult", "extra")

    def __init__(self, rt, delta, norm, mult, extra=None):
        self.rt, self.delta, self.norm, self.mult, self.extra = rt, delta, norm, float(mult), extra

    def also_add(self, extra):
        """The same with one more float32 addend of x's shape."""
        if self.extra is not None:
            raise ValueError("a normed delta carries one extra addend")
        return NormedDelta(self.rt, self.delta, self.norm, self.mult, extra)

    def run(self):
        import torch
        out = self.norm.forward(self.delta, torch.float32, scale=self.mult)
        if self.extra is not None:
            self.rt.ops.residual_add(out, self.extra)
        return out

    def add_to(self, x, next_norm=None, out=None):
        n = self.norm
        return self.rt.ops.sandwich_step(x, self.delta, n.weight, n.bias, n.spec.eps, self.mult, self.extra,
                                         next_norm.weight if next_norm is not None else None,
                                         next_norm.bias if next_norm is not None else None,
                                         next_norm.spec.eps if next_norm is not None else 0.0, out)


@register("norm", "layer_norm")
class LayerNorm:
    """y = (x - mean x) / sqrt(var x + eps) * w + b, in float32."""

    graph_safe = True   # forward launches kernels only: no host reads, no data-dependent launches
    fuses_products = True       # add_forward takes pending deltas of any kind

    def __init__(self, spec, runtime):
        self.spec = spec
        self.rt = runtime
        self.weight = self.bias = None

    @staticmethod
    def params(spec):
        return {spec.name: ParamSpec((spec.width,), "float", ("one_plus_normal", 0.05)),
                spec.bias_name: ParamSpec((spec.width,), "float", ("normal", 0.05))}

    @staticmethod
    def placement(spec):
        return {spec.name: "float32", spec.bias_name: "float32"}

    @staticmethod
    def variants(spec, dtype):
        return [("layer_norm", None)]

    def load(self, tensors):
        self.weight, self.bias = tensors[self.spec.name], tensors[self.spec.bias_name]

    def forward(self, x, out_dtype, scale=1.0):
        """`x` may come in slabs [parts, rows, width]."""
        return self.rt.ops.layer_norm(x, self.weight, self.bias, self.spec.eps, self.rt.empty(tuple(x.shape[-2:]), out_dtype), scale=scale)

    def add_forward(self, x, delta, out_dtype):
        if isinstance(delta, NormedDelta):
            return delta.add_to(x, self, self.rt.empty(x.shape, out_dtype))
        self.rt.ops.residual_add(x, self.rt.settle(delta))
        return self.forward(x, out_dtype)

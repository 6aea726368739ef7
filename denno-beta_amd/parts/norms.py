"""Norms."""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.spec import ParamSpec
from .base import NORMS, Part


@NORMS.register("layernorm")
class LayerNorm(Part):
    """(x - mean) / sqrt(var + eps) * weight + bias, statistics and affine in 32-bit
    (crates/denno-engine/src/tensor.rs:1101-1112)."""
    graph_safe = True

    def __init__(self, width: int, eps: float, weight_name: str, bias_name=None):
        self.width, self.eps = width, eps
        self.weight_name, self.bias_name = weight_name, bias_name

    def param_specs(self):
        specs = [ParamSpec(self.weight_name, (self.width,), "vector", ("normal", 1.0, 0.02))]
        if self.bias_name:
            specs.append(ParamSpec(self.bias_name, (self.width,), "vector", ("normal", 0.0, 0.01)))
        return specs

    def bind(self, tensors, runtime):
        super().bind(tensors, runtime)
        self.weight = tensors[self.weight_name]
        self.bias = tensors[self.bias_name] if self.bias_name else None

    def fused_params(self):
        """What a kernel that runs this norm itself needs (parts.base.LazyNorm)."""
        return ("layernorm", self.weight, self.bias, self.eps)

    adds_deferred = True      # forward(..., deferred=): its kernel first adds a product's sum into the rows (parts.base.DeferredSum)

    def forward(self, x, out_dtype, rows=None, packed=False, deferred=None):
        n = x.shape[0] if rows is None else rows.shape[0]
        if packed:
            out = ops.packed_rows(n, self.width, x.device)
        else:
            out = torch.empty((n, self.width), dtype=out_dtype, device=x.device)
        if deferred is not None and deferred.filled:
            if rows is None and self.width <= 8192:
                part, bias = deferred.part, deferred.bias
                deferred.part = deferred.bias = None
                return ops.layernorm_join(x, part, bias, self.weight, self.bias, self.eps, out)
            deferred.flush(x)
        return ops.layernorm(x, self.weight, self.bias, self.eps, out, rows)


@NORMS.register("rmsnorm")
class RMSNorm(Part):
    """x / sqrt(mean(x^2) + eps) * weight, eps inside the root, statistics in 32-bit.  one_weight: the checkpoint holds a
    single number (a tensor without dimensions) that multiplies every column."""
    graph_safe = True
    libraries = ("sequence",)

    def __init__(self, width: int, eps: float, weight_name: str, one_weight: bool = False):
        self.width, self.eps, self.weight_name, self.one_weight = width, eps, weight_name, bool(one_weight)

    def param_specs(self):
        return [ParamSpec(self.weight_name, () if self.one_weight else (self.width,), "vector", ("normal", 1.0, 0.1))]

    def bind(self, tensors, runtime):
        super().bind(tensors, runtime)
        self.weight = tensors[self.weight_name]
        if self.one_weight:      # (the kernels take a number per column)
            self.weight = self.weight.reshape(1).expand(self.width).contiguous()

    def forward(self, x, out_dtype, rows=None, packed=False):
        # (packed rows are not written here: the consumer's Linear takes a tensor as well)
        n = x.shape[0] if rows is None else rows.shape[0]
        out = torch.empty((n, self.width), dtype=out_dtype, device=x.device)
        return ops.rmsnorm(x, self.weight, self.eps, out, rows)


@NORMS.register("rmsnorm_into_stream")
class StreamRMSNorm(RMSNorm):
    """The norm that stands behind a mixer or a feed-forward, on the result's way into the stream:
    x += mult * (y / sqrt(mean(y^2) + eps) * weight) * scale, with `scale` a vector of the layer's own (a name, or None)
    and `mult` a constant of the model.  `add_into(y, x)` does it in one kernel (gate: 32-bit rows z; y is y * sigmoid(z)
    before the norm, a gate on the sublayer's result); `forward` is the norm alone."""

    def __init__(self, width: int, eps: float, weight_name: str, scale_name=None, mult: float = 1.0):
        super().__init__(width, eps, weight_name)
        self.scale_name, self.mult = scale_name, float(mult)

    def param_specs(self):
        specs = super().param_specs()
        if self.scale_name:
            specs.append(ParamSpec(self.scale_name, (self.width,), "vector", ("normal", 1.0, 0.2)))
        return specs

    def bind(self, tensors, runtime):
        super().bind(tensors, runtime)
        self.scale = tensors[self.scale_name] if self.scale_name else None

    def add_into(self, y, x, gate=None, then=None, out_dtype=None):
        """then: the norm that reads the stream next; if it is a plain `rmsnorm`, its rows come out of the same kernel and
        are returned (else None, and that norm runs as a kernel of its own)."""
        nxt = following_norm(then, x, out_dtype)
        ops.rmsnorm_add(y, self.weight, self.scale, self.mult, self.eps, x, gate=gate, then=nxt)
        return nxt[2] if nxt is not None else None


def following_norm(norm, x, out_dtype):
    """(weight, eps, rows to fill) for a kernel that, having changed the stream's rows x, norms them for `norm` as well; None
    where `norm` is none or not a plain root-mean-square norm over the whole row."""
    if norm is None or type(norm) is not RMSNorm or norm.width != x.shape[1] or out_dtype is None:
        return None
    return norm.weight, norm.eps, torch.empty(x.shape, dtype=out_dtype, device=x.device)

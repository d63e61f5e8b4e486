"""Norms over the width of a row.

RMSNorm: y = x / sqrt(mean(x^2) + eps) * w; the weight multiplies after the
scale, eps sits inside the root, no 1+w, no bias
(src/alofa/kernels/cpu/scalar.mojo:93-129)."""
from __future__ import annotations

from .. import ops
from ..weights.loader import TensorRule
from .base import Norm, register_part


class RMSNorm(Norm):
    """params: name (tensor name), width, eps; scalar (True: the weight is one number for all channels, a tensor without
    dimensions; it is spread over the width when the weights are loaded, so every kernel that takes an RMSNorm takes this one)."""

    @classmethod
    def tensors(cls, spec):
        return {spec.params["name"]: TensorRule(() if spec.params.get("scalar", False) else (spec.params["width"],), "norm")}

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        self.eps = float(spec.params["eps"])
        self.width = int(spec.params["width"])
        weight = weights[spec.params["name"]]
        self.weight = rt.vector(weight.float().reshape(1).repeat(self.width) if spec.params.get("scalar", False) else weight)

    def as_rmsnorm(self):
        return self.weight, self.eps

    def forward(self, out, x, rows=None):
        ops.rmsnorm(out, x, self.weight, self.eps, self.rt.exact, rows)


register_part("norm", "rmsnorm", RMSNorm)


class LayerNorm(Norm):
    """y = (x - mean) / sqrt(var + eps) * w + b with var the mean of the squared deviations; float32 arithmetic.
    params: name (the weight's tensor name), bias (the bias's), width, eps."""

    @classmethod
    def tensors(cls, spec):
        p = spec.params
        return {p["name"]: TensorRule((p["width"],), "norm"), p["bias"]: TensorRule((p["width"],), "bias")}

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        self.eps = float(spec.params["eps"])
        self.width = int(spec.params["width"])
        self.weight = rt.vector(weights[spec.params["name"]])
        self.bias = rt.vector(weights[spec.params["bias"]])

    def as_layernorm(self):
        return self.weight, self.bias, self.eps

    def forward(self, out, x, rows=None):
        ops.layernorm(out, x, self.weight, self.bias, self.eps, self.rt.exact, rows)


register_part("norm", "layernorm", LayerNorm)

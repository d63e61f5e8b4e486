"""Dense feed-forwards.

SwiGLU: down(silu(gate(x)) * up(x)), no biases; silu is
x / (1 + exp(-x)) (src/alofa/kernels/cpu/scalar.mojo:219-231,
src/alofa/engine/executor.mojo:806-837). Gate and up run as one kernel that
applies the activation before anything is written.

Two matrices with an activation between them: down(act(up(x))), no biases. The activation xIELU has two numbers
p, q of its own per layer: z > 0: softplus(p) z^2 + z/2; z <= 0: (1/2 + softplus(q)) (exp(z) - 1 - z) + z/2. The
activation relu_squared is max(z, 0)^2 and has no tensor of its own; gelu_tanh is z/2 (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3))).
Both matrices may have biases."""
from __future__ import annotations

import math

import torch

from .. import ops
from ..errors import AlofaError
from ..weights.loader import TensorRule
from .base import FeedForward, register_part


class SwiGLU(FeedForward):
    """params: prefix, hidden, intermediate."""
    capturable = True   # native kernels on the current stream only: a decode step may be graph-captured

    @classmethod
    def tensors(cls, spec):
        p = spec.params
        pre, h, i = p["prefix"], p["hidden"], p["intermediate"]
        return {pre + "gate_proj.weight": TensorRule((i, h)), pre + "up_proj.weight": TensorRule((i, h)),
                pre + "down_proj.weight": TensorRule((h, i))}

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        p = spec.params
        self.hidden, self.intermediate = int(p["hidden"]), int(p["intermediate"])
        pre = p["prefix"]
        gate, up = weights[pre + "gate_proj.weight"], weights[pre + "up_proj.weight"]
        if gate.dtype is not up.dtype:
            gate, up = gate.float(), up.float()
        self.w_gate, self.w_up = rt.matrix(gate), rt.matrix(up)
        self.w_down = rt.matrix(weights[pre + "down_proj.weight"])

    def fuses_norm(self, norm, rows):
        return (not self.rt.exact and norm.as_rmsnorm() is not None
                and ops.can_fuse_norm(rows, self.w_gate, self.rt.dtype, swiglu=True))

    gives_normed = True

    def forward(self, ctx, x, residual, norm=None, then=None):
        act = ctx.scratch("ff_act", (residual.shape[0], self.intermediate), self.rt.dtype)
        if norm is not None:      # the norm before the feed-forward rides on the gate/up product
            ops.gemm_swiglu(act, residual, self.w_gate, self.w_up, norm=norm.as_rmsnorm())
        else:
            ops.gemm_swiglu(act, x, self.w_gate, self.w_up, exact=self.rt.exact)
        then_norm = None
        if then is not None:      # the norm behind this part, left in the rows given with it
            weight, eps = then[0].as_rmsnorm()
            then_norm = (weight, eps, then[1])
        ops.gemm(residual, act, self.w_down, add_to_out=True, exact=self.rt.exact, then_norm=then_norm)


def _softplus(z: float) -> float:
    return math.log1p(math.exp(-abs(z))) + max(z, 0.0)


class DenseActivated(FeedForward):
    """params: prefix, hidden, intermediate, activation ("xielu", "relu_squared" or "gelu_tanh"), names (after the prefix: up, down, act for
    xielu, and up_bias, down_bias where ``biases`` is set). ``forward(..., scale=)`` with a float32 vector: what is added to the stream is
    multiplied by it channel by channel; ``then=`` (weight, eps, rows): the RMSNorm of the stream's new rows is left in ``rows``."""
    capturable = True
    takes_channel_scale = True

    @classmethod
    def tensors(cls, spec):
        p = spec.params
        pre, h, i, names = p["prefix"], p["hidden"], p["intermediate"], p["names"]
        out = {pre + names["up"]: TensorRule((i, h), "fan_in"), pre + names["down"]: TensorRule((h, i), "fan_in")}
        if p.get("activation", "xielu") == "xielu":
            out[pre + names["act"]] = TensorRule((2,), "bias")
        if p.get("biases", False):
            out.update({pre + names["up_bias"]: TensorRule((i,), "bias"), pre + names["down_bias"]: TensorRule((h,), "bias")})
        return out

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        p = spec.params
        self.activation = p.get("activation", "xielu")
        if self.activation not in ("xielu", "relu_squared", "gelu_tanh"):
            raise AlofaError("unsupported", "no such activation is built", f"activation={p['activation']}")
        self.hidden, self.intermediate = int(p["hidden"]), int(p["intermediate"])
        pre, names = p["prefix"], p["names"]
        self.w_up, self.w_down = rt.matrix(weights[pre + names["up"]]), rt.matrix(weights[pre + names["down"]])
        self.b_up = self.b_down = None
        if p.get("biases", False):
            self.b_up, self.b_down = rt.vector(weights[pre + names["up_bias"]]), rt.vector(weights[pre + names["down_bias"]])
        if self.activation == "xielu":
            # the two numbers are fixed once the weights are: what the kernel needs of them is formed here, in float64
            pq = weights[pre + names["act"]].double().tolist()
            self.a, self.b = _softplus(pq[0]), 0.5 + _softplus(pq[1])

    def fuses_norm(self, norm, rows):
        return not self.rt.exact and norm.as_rmsnorm() is not None and ops.can_fuse_norm(rows, self.w_up, self.rt.dtype)

    def forward(self, ctx, x, residual, scale=None, norm=None, then=None):
        act = ctx.scratch("ff_act", (residual.shape[0], self.intermediate), self.rt.dtype)
        if norm is not None:      # the norm in front rides on the product
            ops.gemm(act, residual, self.w_up, self.b_up, norm=norm.as_rmsnorm())
        else:
            ops.gemm(act, x, self.w_up, self.b_up, exact=self.rt.exact)
        if self.activation == "xielu":
            ops.activation(act, act, ops.XIELU, self.a, self.b, self.rt.exact)
        elif self.activation == "gelu_tanh":
            ops.activation(act, act, ops.GELU_TANH, exact=self.rt.exact)
        else:
            ops.relu_squared(act, act)
        if scale is None and self.b_down is None:
            ops.gemm(residual, act, self.w_down, add_to_out=True, exact=self.rt.exact)
            if then is not None:
                ops.rmsnorm(then[2], residual, then[0], then[1], self.rt.exact)
        elif scale is None:
            apart = ctx.scratch("sub_out", tuple(residual.shape), torch.float32)
            ops.gemm(apart, act, self.w_down, self.b_down, exact=self.rt.exact)
            ops.add_scaled(residual, apart, 1.0, exact=self.rt.exact)
            if then is not None:
                ops.rmsnorm(then[2], residual, then[0], then[1], self.rt.exact)
        else:
            ops.gemm_channel_scaled(residual, act, self.w_down, scale, ctx.scratch("sub_out", tuple(residual.shape), torch.float32), self.rt.exact, then_norm=then,
                                    bias=self.b_down)


register_part("feed_forward", "swiglu", SwiGLU)
register_part("feed_forward", "dense_activated", DenseActivated)

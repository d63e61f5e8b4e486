"""Feed-forwards of which a token takes a few: a router scores the experts, the token takes the best ``top`` of them, and
what they give is summed with weights that follow from the scores; an expert that every token takes may stand beside them.

Router: z = x W_r^T in float32; the score is sigmoid(z); the ``top`` largest are taken (the lower index among equals);
the weights are the taken scores (made to sum to one first where the design says so) times ``weight_scale``.
Expert ("clamped_glu"): a = min(gate(x), limit), b = clamp(up(x), -limit, limit); down(a sigmoid(slope a) (b + 1)).

Another router ("softmax"): the score is softmax(z) over all experts; the choice goes by score + ``correction`` (a tensor), within the
``groups.keep`` best of ``groups.count`` groups of neighbouring experts (a group's score: its largest member's); the weights are the
scores themselves. The last ``passing`` experts of such a router have no matrices: they hand the row on, times their weight.
Another expert ("silu_glu"): down(silu(gate(x)) up(x)).

The experts' matrices lie side by side in one tensor each (gate and up by rows, down by columns, the shared expert's
last), so that every expert is a slice of them."""
from __future__ import annotations

import os

import torch

from .. import ops
from ..errors import AlofaError
from ..weights.loader import TensorRule
from .base import FeedForward, register_part


SPARSE_EXPERTS = os.environ.get("ALOFA_SPARSE_EXPERTS", "1") != "0"      # 0 (for measurements): every expert against every row


class RoutedExperts(FeedForward):
    """params: prefix, hidden, experts, top, score ("sigmoid"), weight_scale, renormalize, expert {intermediate, limit},
    shared (the same, or None), activation ("clamped_glu"), slope, names (after the prefix: router; expert, a pattern with {}
    for the expert's number; shared; gate, up, down after an expert's name and a dot).
    Optional: correction (a tensor's name after the prefix, [experts + passing]), groups {count, keep}, passing (experts without
    matrices behind the others; the router has experts + passing outputs), router_init (the rule random router weights are drawn by).
    ``forward(..., scale=)`` with a float32 vector: what is added to the stream is multiplied by it channel by channel;
    ``forward(..., out=)``: the result is stored there (float32, the stream's shape) and the stream left alone."""
    capturable = True
    takes_channel_scale = True

    @staticmethod
    def _expert_names(p, e) -> dict:
        n = p["names"]
        stem = p["prefix"] + (n["shared"] if e is None else n["expert"].format(e)) + "."
        return {k: stem + n[k] for k in ("gate", "up", "down")}

    @classmethod
    def tensors(cls, spec):
        p = spec.params
        h = p["hidden"]
        out = {}
        for e in range(p["experts"]):
            names, i = cls._expert_names(p, e), p["expert"]["intermediate"]
            out.update({names["gate"]: TensorRule((i, h), "fan_in"), names["up"]: TensorRule((i, h), "fan_in"), names["down"]: TensorRule((h, i), "fan_in")})
        out[p["prefix"] + p["names"]["router"]] = TensorRule((p["experts"] + int(p.get("passing", 0)), h), p.get("router_init", "fan_in"))
        if p.get("correction") is not None:
            out[p["prefix"] + p["correction"]] = TensorRule((p["experts"] + int(p.get("passing", 0)),), "bias")
        if p.get("shared") is not None:
            names, i = cls._expert_names(p, None), p["shared"]["intermediate"]
            out.update({names["gate"]: TensorRule((i, h), "fan_in"), names["up"]: TensorRule((i, h), "fan_in"), names["down"]: TensorRule((h, i), "fan_in")})
        return out

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        p = spec.params
        self.score, self.activation = p.get("score", "sigmoid"), p.get("activation", "clamped_glu")
        if self.score not in ("sigmoid", "softmax") or self.activation not in ("clamped_glu", "silu_glu"):
            raise AlofaError("unsupported", "no such router score or expert activation is built", f"score={p.get('score')} activation={p.get('activation')}")
        self.hidden, self.experts, self.top = int(p["hidden"]), int(p["experts"]), int(p["top"])
        self.passing = int(p.get("passing", 0))
        groups = p.get("groups") or {"count": 1, "keep": 1}
        self.groups, self.keep = int(groups["count"]), int(groups["keep"])
        routed = self.experts + self.passing
        if not 0 < self.top <= routed <= ops.MAX_EXPERTS or self.experts <= 0 or self.passing < 0:
            raise AlofaError("unsupported", f"a token takes 1..experts experts of at most {ops.MAX_EXPERTS}", f"experts={self.experts} passing={self.passing} top={self.top}")
        if self.score == "sigmoid" and (self.passing or self.groups != 1 or p.get("correction") is not None):
            raise AlofaError("unsupported", "groups, a correction and experts without matrices go with the softmax router", f"score={self.score}")
        if self.groups < 1 or routed % self.groups or not 1 <= self.keep <= self.groups or self.top > self.keep * (routed // self.groups):
            raise AlofaError("invalid_argument", "equal groups, of which the kept ones hold at least the experts a token takes", f"experts={routed} groups={self.groups} keep={self.keep} top={self.top}")
        self.weight_scale, self.renormalize, self.slope = float(p.get("weight_scale", 1.0)), bool(p.get("renormalize", False)), float(p.get("slope", 1.0))
        # silu(g) u is the clamped form without limits, with slope one and nothing added to u
        unbounded = self.activation == "silu_glu"
        self.offset = 0.0 if unbounded else 1.0
        self.ff, self.limit = int(p["expert"]["intermediate"]), float("inf") if unbounded else float(p["expert"]["limit"])
        shared = p.get("shared")
        self.shared_ff, self.shared_limit = (int(shared["intermediate"]), float("inf") if unbounded else float(shared["limit"])) if shared is not None else (0, 0.0)
        self.correction = rt.vector(weights[p["prefix"] + p["correction"]]) if p.get("correction") is not None else None
        who = list(range(self.experts)) + ([None] if shared is not None else [])
        names = [self._expert_names(p, e) for e in who]
        self.w_gate = rt.matrix(torch.cat([weights[n["gate"]] for n in names], dim=0))
        self.w_up = rt.matrix(torch.cat([weights[n["up"]] for n in names], dim=0))
        self.w_down = rt.matrix(torch.cat([weights[n["down"]] for n in names], dim=1))
        self.w_router = rt.matrix(weights[p["prefix"] + p["names"]["router"]])
        self.channels = self.experts * self.ff + self.shared_ff

    def route(self, ctx, x):
        """(dense [T, E], chosen [T, top], weights [T, top], and, with experts that hand the row on, their summed weight [T] or None) of the step's rows."""
        T = x.shape[0]
        z = ctx.scratch("router_z", (T, self.experts + self.passing), torch.float32)
        ops.gemm(z, x, self.w_router, exact=self.rt.exact)
        dense = ctx.scratch("router_dense", (T, self.experts), torch.float32)
        chosen, weights = ctx.scratch("router_chosen", (T, self.top), torch.int32), ctx.scratch("router_weights", (T, self.top), torch.float32)
        if self.score == "sigmoid":
            ops.route_top(z, dense, chosen, weights, self.top, self.weight_scale, self.renormalize, self.rt.exact)
            return dense, chosen, weights, None
        passed = ctx.scratch("router_passed", (T,), torch.float32)
        ops.route_groups(z, self.correction, dense, chosen, weights, passed, self.top, self.passing, self.groups, self.keep, self.weight_scale,
                         self.renormalize, self.rt.exact)
        return dense, chosen, weights, passed if self.passing else None

    def sparse(self, x) -> bool:
        """Whether the experts run slot by slot (every row against the experts it takes only) rather than all of them against
        every row with weights of zero: where a token leaves at least half of the experts out, and the kernel takes the sizes."""
        return (SPARSE_EXPERTS and not self.rt.exact and 2 * self.top <= self.experts
                and ops.can_group_experts(x, self.w_gate, self.ff, self.shared_ff))

    def forward(self, ctx, x, residual, scale=None, out=None):
        T, exact = residual.shape[0], self.rt.exact
        dense, chosen, weights, passed = self.route(ctx, x)
        if passed is not None and scale is not None:
            raise AlofaError("unsupported", "experts that hand the row on do not go with a channel scale")
        if self.sparse(x):
            rows = ops.ExpertRows(T, self.top, self.experts, self.shared_ff > 0, ctx.scratch)
            ops.expert_rows(rows, chosen, weights)
            act = ctx.scratch("experts_act", (rows.slots, (max(self.ff, self.shared_ff) + 7) // 8 * 8), torch.bfloat16)
            ops.experts_gate_up(act, x, self.w_gate, self.w_up, rows, self.ff, self.shared_ff, self.limit, self.shared_limit, self.slope, self.offset)
            y = ctx.scratch("experts_out", (rows.slots, self.hidden), torch.float32)
            ops.experts_down(y, act, self.w_down, rows, self.ff, self.shared_ff)
            ops.experts_sum(residual if out is None else out, y, rows, scale, passed=None if passed is None else (passed, x), assign=out is not None)
            return
        # every expert's gate and up for every row, the rows an expert is not taken by weighted with zero
        g, u = ctx.scratch("experts_gate", (T, self.channels), self.rt.dtype), ctx.scratch("experts_up", (T, self.channels), self.rt.dtype)
        ops.gemm(g, x, self.w_gate, exact=exact)
        ops.gemm(u, x, self.w_up, exact=exact)
        act = ctx.scratch("ff_act", (T, self.channels), self.rt.dtype)
        ops.clamped_glu(act, g, u, dense, self.experts, self.ff, self.shared_ff, self.limit, self.shared_limit, self.slope, exact, self.offset)
        if out is not None:
            ops.gemm(out, act, self.w_down, exact=exact)
            if scale is not None:
                out.mul_(scale)
            if passed is not None:
                ops.add_row_scaled(out, x, passed, exact)
        elif scale is None:
            ops.gemm(residual, act, self.w_down, add_to_out=True, exact=exact)
            if passed is not None:
                ops.add_row_scaled(residual, x, passed, exact)
        else:
            ops.gemm_channel_scaled(residual, act, self.w_down, scale, ctx.scratch("sub_out", tuple(residual.shape), torch.float32), exact)


register_part("feed_forward", "routed_experts", RoutedExperts)

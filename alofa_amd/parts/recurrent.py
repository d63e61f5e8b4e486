"""Mixers that keep a state of fixed size per request instead of keys: per head a matrix S [dk, dv] in float32 that
every token decays and adds to, S_t = diag(w_t) S_(t-1) + k_t v_t^T, and reads out with its query. They differ in
where the decay comes from and in the order of read-out and update; the recurrence itself is one kernel
(``ops.linear_recurrence``), and so are the norm of every head's read-out with the gate (``ops.headnorm_gate``).

retention       w = a constant per head; rotary positions on q and k; k scaled by dk^(-1/2); o_t = S_t^T q_t;
                o / rms(o) per head, times silu(gate), output projection.
gated_linear    w_t = sigmoid(z_t)^(1/tau) per key channel, z = W_a2 (W_a1 x) + b; q scaled by dk^(-1/2); o_t = S_t^T q_t;
                RMS norm per head with a weight shared by the heads, times silu(gate), output projection.
time_mix        RWKV-style: each of r, k, v, g, w reads its own mix of the token with the one before it,
                x + (x' - x) mu_s; w_t = exp(-exp(W_w2 tanh(W_w1 mix_w) + w0)); o_t = (S_(t-1) + diag(u) k_t v_t^T)^T r_t,
                then the update; o / rms(o) per head, times a weight per channel, times silu(g), output projection.

lightning_attention  w = a constant per head; q, k, v through silu; o_t = S_t^T q_t; the heads together through an RMS norm with a
                weight, times sigmoid(gate), output projection.
matrix_memory   exponential gates per head kept in range by a running maximum m (state beside S): i = cap tanh(zi / cap),
                f = log sigmoid(cap tanh(zf / cap)), m_t = max(f + m_(t-1), i); S_t = exp(f + m_(t-1) - m_t) S_(t-1) + exp(i - m_t) k v^T, a
                normaliser n_t likewise with k alone; o = S_t^T q / (max(|n_t . q|, exp(-m_t)) + 1e-6), q scaled by dk^(-1/2); o / rms(o)
                per head, times a weight per channel, times sigmoid(gate), output projection.

state_space     a decay per head and step made of a step size (the "state-space duality" form): one projection gives z, x, B, C and dt side by side;
                x, B, C pass a short causal convolution with bias and silu; dt = softplus(dt + bias); S_t = exp(-exp(A_log) dt_t) S_(t-1) + dt_t B_t x_t^T
                (S [state, value_dim] per head; B and C shared by the heads of a group), y_t = S_t^T C_t + D x_t; y times silu(z), an RMS norm over
                each of several equal parts of the row, a weight, output projection. The convolution's last inputs are a second piece of state.

Projections and gates run in the activation dtype; decays, the state, the read-out and the head norms in float32.
Every one of them takes ``out=`` (see ``Mixer.forward``)."""
from __future__ import annotations

import torch

from .. import ops
from ..config.base import PartSpec
from ..errors import AlofaError
from ..weights.loader import TensorRule
from .attention import _padded_heads
from .base import Mixer, StateNeed, TimeConv, build_part, part_class, register_part
from .rows import rows_of_requests


def _stacked(rt, mats: list) -> torch.Tensor:
    if len({m.dtype for m in mats}) > 1:
        mats = [m.float() for m in mats]
    return rt.matrix(torch.cat(mats, dim=0))


class RecurrentMixer(Mixer):
    """What the three kinds share: sizes, the state, the way out (head norm, gate, output projection)."""
    capturable = True   # native kernels on the current stream only: a decode step may be graph-captured

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        p = spec.params
        self.hidden, self.heads, self.dk = int(p["hidden"]), int(p["heads"]), int(p["key_dim"])
        self.dv = int(p.get("value_dim") or self.dk)
        self.eps = float(p["eps"])
        if self.heads <= 0 or self.dv <= 0 or not 0 < self.dk <= ops.RECURRENCE_MAX_KEYS:
            raise AlofaError("unsupported", f"the recurrence kernel takes key sizes up to {ops.RECURRENCE_MAX_KEYS}", f"heads={self.heads} key_dim={self.dk} value_dim={self.dv}")

    def state_need(self):
        return StateNeed((self.heads, self.dk, self.dv), torch.float32)

    def _readouts(self, ctx, rows: int):
        """Room for the read-outs of a step: float32 [parts, T, heads * dv]; a step of many rows may leave them in parts."""
        return ctx.scratch("recurrent_out", (ops.recurrence_max_parts(self.dk), rows, self.heads * self.dv), torch.float32)

    def _leave(self, ctx, o, parts, gate, weight, residual, out):
        """Head norm, gate and output projection of the read-outs ``o`` (float32 [P, T, heads * dv], the first ``parts`` to be added)."""
        y = ctx.scratch("recurrent_gated", (o.shape[1], self.heads * self.dv), self.rt.dtype)
        ops.headnorm_gate(y, o, gate, weight, self.heads, self.dv, self.eps, self.rt.exact, parts=parts)
        if out is not None:
            ops.gemm(out, y, self.w_o, exact=self.rt.exact)
        else:
            ops.gemm(residual, y, self.w_o, add_to_out=True, exact=self.rt.exact)


class Retention(RecurrentMixer):
    """params: prefix, hidden, heads, key_dim, value_dim, decay (one per head), position (PartSpec, for heads of
    key_dim), eps. Tensors: prefix + q, k, v, g, o."""

    @classmethod
    def tensors(cls, spec):
        p = spec.params
        pre, h, kd, vd = p["prefix"], p["hidden"], p["heads"] * p["key_dim"], p["heads"] * (p.get("value_dim") or p["key_dim"])
        return {pre + "q": TensorRule((kd, h), "fan_in"), pre + "k": TensorRule((kd, h), "fan_in"), pre + "v": TensorRule((vd, h), "fan_in"),
                pre + "g": TensorRule((vd, h), "fan_in"), pre + "o": TensorRule((h, vd), "fan_in")}

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        p, pre = spec.params, spec.params["prefix"]
        decay = [float(x) for x in p["decay"]]
        if len(decay) != self.heads:
            raise AlofaError("invalid_argument", "retention takes one decay per head", f"heads={self.heads} decays={len(decay)}")
        self.decay = torch.tensor(decay, dtype=torch.float32, device=rt.device)
        self.k_scale = float(self.dk) ** -0.5
        # the rotation pairs channels, so a head of odd size gets one more key channel whose q and k are zero (it adds nothing to any product)
        position, true_dk = p["position"], self.dk
        if self.dk % 2:
            self.dk += 1
            position = part_class("position", position.kind).for_head(position, self.dk)
        self.position = build_part("position", position, weights, rt)
        order = self.position.channel_order()
        self.w_in = _stacked(rt, [_padded_heads(weights[pre + "q"], self.heads, true_dk, self.dk, order), _padded_heads(weights[pre + "k"], self.heads, true_dk, self.dk, order),
                                  weights[pre + "v"], weights[pre + "g"]])
        self.w_o = rt.matrix(weights[pre + "o"])
        self.capturable = self.position.table(1) is not None

    def prepare(self, n_positions):
        self.position.table(n_positions)

    def forward(self, ctx, where, x, residual, out=None):
        T, kd, vd = x.shape[0], self.heads * self.dk, self.heads * self.dv
        proj = ctx.scratch("recurrent_proj", (T, 2 * kd + 2 * vd), self.rt.dtype)
        ops.gemm(proj, x, self.w_in, exact=self.rt.exact)
        table = self.position.table(ctx.n_positions)
        if table is None:
            self.position.apply(ctx, proj[:, :kd].unflatten(1, (self.heads, self.dk)), proj[:, kd:2 * kd].unflatten(1, (self.heads, self.dk)))
        else:      # queries and keys alike: 2 * heads heads to rotate, nothing to write to pages
            ops.rope_kv_write(proj, table[0], table[1], ctx.positions, 2 * self.heads, 0, self.dk)
        o = self._readouts(ctx, T)
        parts = ops.linear_recurrence(o, proj[:, :kd], proj[:, kd:2 * kd], proj[:, 2 * kd:2 * kd + vd], ctx.state(where), rows_of_requests(ctx),
                                      self.heads, self.dk, self.dv, ops.DECAY_PER_HEAD, self.decay, k_scale=self.k_scale)
        self._leave(ctx, o, parts, proj[:, 2 * kd + vd:], None, residual, out)


class GatedLinearAttention(RecurrentMixer):
    """params: prefix, hidden, heads, key_dim, value_dim, tau, rank (of the decay's two-step projection), eps.
    Tensors: prefix + q, k, v, g, o, a1 [rank, hidden], a2 [heads * key_dim, rank], a2.b, norm [value_dim]."""

    @classmethod
    def tensors(cls, spec):
        p = spec.params
        dv = p.get("value_dim") or p["key_dim"]
        pre, h, kd, vd, r = p["prefix"], p["hidden"], p["heads"] * p["key_dim"], p["heads"] * dv, p["rank"]
        return {pre + "q": TensorRule((kd, h), "fan_in"), pre + "k": TensorRule((kd, h), "fan_in"), pre + "v": TensorRule((vd, h), "fan_in"),
                pre + "g": TensorRule((vd, h), "fan_in"), pre + "o": TensorRule((h, vd), "fan_in"), pre + "norm": TensorRule((dv,), "norm"),
                pre + "a1": TensorRule((r, h), "fan_in"), pre + "a2": TensorRule((kd, r), "fan_in"), pre + "a2.b": TensorRule((kd,), "decay_bias")}

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        p, pre = spec.params, spec.params["prefix"]
        self.tau, self.rank = float(p["tau"]), int(p["rank"])
        if not self.tau > 0:
            raise AlofaError("invalid_argument", "tau must be positive", f"tau={self.tau}")
        self.w_in = _stacked(rt, [weights[pre + n] for n in ("q", "k", "v", "g", "a1")])
        self.w_a2, self.b_a2 = rt.matrix(weights[pre + "a2"]), rt.vector(weights[pre + "a2.b"])
        self.w_o = rt.matrix(weights[pre + "o"])
        self.norm = rt.vector(weights[pre + "norm"].float().repeat(self.heads))      # one weight per value channel, the same for every head
        self.q_scale = float(self.dk) ** -0.5

    def forward(self, ctx, where, x, residual, out=None):
        T, kd, vd = x.shape[0], self.heads * self.dk, self.heads * self.dv
        proj = ctx.scratch("recurrent_proj", (T, 2 * kd + 2 * vd + self.rank), self.rt.dtype)
        ops.gemm(proj, x, self.w_in, exact=self.rt.exact)
        z = ctx.scratch("recurrent_decay", (T, kd), torch.float32)
        ops.gemm(z, proj[:, 2 * kd + 2 * vd:], self.w_a2, self.b_a2, exact=self.rt.exact)
        o = self._readouts(ctx, T)
        parts = ops.linear_recurrence(o, proj[:, :kd], proj[:, kd:2 * kd], proj[:, 2 * kd:2 * kd + vd], ctx.state(where), rows_of_requests(ctx),
                                      self.heads, self.dk, self.dv, ops.DECAY_SIGMOID_ROOT, z, tau=self.tau, q_scale=self.q_scale)
        self._leave(ctx, o, parts, proj[:, 2 * kd + vd:2 * kd + 2 * vd], self.norm, residual, out)


class LightningAttention(RecurrentMixer):
    """params: prefix, hidden, heads, key_dim, value_dim, decay (one per head), eps. Tensors: prefix + q, k, v, g, o, norm [heads * value_dim]."""

    @classmethod
    def tensors(cls, spec):
        p = spec.params
        pre, h, kd, vd = p["prefix"], p["hidden"], p["heads"] * p["key_dim"], p["heads"] * (p.get("value_dim") or p["key_dim"])
        return {pre + "q": TensorRule((kd, h), "fan_in"), pre + "k": TensorRule((kd, h), "fan_in"), pre + "v": TensorRule((vd, h), "fan_in"),
                pre + "g": TensorRule((vd, h), "fan_in"), pre + "o": TensorRule((h, vd), "fan_in"), pre + "norm": TensorRule((vd,), "norm")}

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        p, pre = spec.params, spec.params["prefix"]
        decay = [float(x) for x in p["decay"]]
        if len(decay) != self.heads:
            raise AlofaError("invalid_argument", "one decay per head", f"heads={self.heads} decays={len(decay)}")
        self.decay = torch.tensor(decay, dtype=torch.float32, device=rt.device)
        self.w_in = _stacked(rt, [weights[pre + n] for n in ("q", "k", "v", "g")])
        self.w_o = rt.matrix(weights[pre + "o"])
        self.norm = rt.vector(weights[pre + "norm"])

    def forward(self, ctx, where, x, residual, out=None):
        T, kd, vd = x.shape[0], self.heads * self.dk, self.heads * self.dv
        proj = ctx.scratch("recurrent_proj", (T, 2 * kd + 2 * vd), self.rt.dtype)
        ops.gemm(proj, x, self.w_in, exact=self.rt.exact)
        qkv = proj[:, :2 * kd + vd]
        ops.activation(qkv, qkv, ops.SILU, exact=self.rt.exact)
        o = self._readouts(ctx, T)
        parts = ops.linear_recurrence(o, proj[:, :kd], proj[:, kd:2 * kd], proj[:, 2 * kd:2 * kd + vd], ctx.state(where), rows_of_requests(ctx),
                                      self.heads, self.dk, self.dv, ops.DECAY_PER_HEAD, self.decay)
        # (the heads together are one row to norm: a "head" of heads * dv channels)
        y = ctx.scratch("recurrent_gated", (T, vd), self.rt.dtype)
        ops.headnorm_gate(y, o, proj[:, 2 * kd + vd:], self.norm, 1, vd, self.eps, self.rt.exact, parts=parts, gate_kind="sigmoid")
        if out is not None:
            ops.gemm(out, y, self.w_o, exact=self.rt.exact)
        else:
            ops.gemm(residual, y, self.w_o, add_to_out=True, exact=self.rt.exact)


class GateMaximum(Mixer):
    """The running maximum of a memory's gates: one float per head and request, beside the memory itself."""
    capturable = True

    def __init__(self, heads: int, rt):
        self.heads, self.rt, self.spec = heads, rt, None

    def state_need(self):
        return StateNeed((self.heads,), torch.float32)


class MatrixMemory(RecurrentMixer):
    """params: prefix, hidden, heads, key_dim, value_dim, gate_cap, eps. Tensors: prefix + q, k, v, g, o, norm [heads * value_dim],
    i [heads, hidden], i.b [heads], f, f.b.

    The normaliser rides through the recurrence as one more value channel that is always one, so the state of a head is
    [key_dim, value_dim + 1]; the gates' running maximum is a second piece of state."""

    @classmethod
    def tensors(cls, spec):
        p = spec.params
        H = p["heads"]
        pre, h, kd, vd = p["prefix"], p["hidden"], H * p["key_dim"], H * (p.get("value_dim") or p["key_dim"])
        return {pre + "q": TensorRule((kd, h), "fan_in"), pre + "k": TensorRule((kd, h), "fan_in"), pre + "v": TensorRule((vd, h), "fan_in"),
                pre + "g": TensorRule((vd, h), "fan_in"), pre + "o": TensorRule((h, vd), "fan_in"), pre + "norm": TensorRule((vd,), "norm"),
                pre + "i": TensorRule((H, h), "fan_in"), pre + "i.b": TensorRule((H,), "bias"), pre + "f": TensorRule((H, h), "fan_in"), pre + "f.b": TensorRule((H,), "gate_bias")}

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        p, pre = spec.params, spec.params["prefix"]
        self.cap = float(p["gate_cap"])
        if not self.cap > 0:
            raise AlofaError("invalid_argument", "the gates' cap is positive", f"gate_cap={self.cap}")
        self.w_in = _stacked(rt, [weights[pre + n] for n in ("q", "k", "v", "g")])
        self.w_gates = _stacked(rt, [weights[pre + "i"], weights[pre + "f"]])
        self.b_gates = rt.vector(torch.cat([weights[pre + "i.b"].float(), weights[pre + "f.b"].float()]))
        self.w_o = rt.matrix(weights[pre + "o"])
        self.norm = rt.vector(weights[pre + "norm"])
        self.q_scale = float(self.dk) ** -0.5
        self.maximum = GateMaximum(self.heads, rt)

    def state_need(self):
        return StateNeed((self.heads, self.dk, self.dv + 1), torch.float32)

    def stateful_parts(self):
        return [self, self.maximum]

    def forward(self, ctx, where, x, residual, out=None):
        T, H, kd, vd = x.shape[0], self.heads, self.heads * self.dk, self.heads * self.dv
        entry, k = where if isinstance(where, tuple) else (where, 0)
        exact, rows = self.rt.exact, rows_of_requests(ctx)
        proj = ctx.scratch("recurrent_proj", (T, 2 * kd + 2 * vd), self.rt.dtype)
        ops.gemm(proj, x, self.w_in, exact=exact)
        z = ctx.scratch("memory_gate_z", (T, 2 * H), torch.float32)
        ops.gemm(z, x, self.w_gates, self.b_gates, exact=exact)
        gates = ctx.scratch("memory_gates", (3, T, H), torch.float32)
        ops.gate_scan(gates, z, ctx.state((entry, k + 1)), rows, H, self.cap)
        qf, kf = ctx.scratch("memory_q", (T, kd), torch.float32), ctx.scratch("memory_k", (T, kd), torch.float32)
        vf, decay = ctx.scratch("memory_v", (T, vd + H), torch.float32), ctx.scratch("recurrent_decay", (T, kd), torch.float32)
        ops.gated_operands(qf, kf, vf, decay, proj[:, :kd], proj[:, kd:2 * kd], proj[:, 2 * kd:2 * kd + vd], gates, H, self.dk, self.dv)
        o = ctx.scratch("memory_out", (ops.recurrence_max_parts(self.dk), T, vd + H), torch.float32)
        parts = ops.linear_recurrence(o, qf, kf, vf, ctx.state((entry, k)), rows, H, self.dk, self.dv + 1, ops.DECAY_GIVEN, decay, q_scale=self.q_scale)
        y = ctx.scratch("recurrent_gated", (T, vd), self.rt.dtype)
        ops.headnorm_gate(y, o, proj[:, 2 * kd + vd:], self.norm, H, self.dv, self.eps, exact, parts=parts, gate_kind="sigmoid", extra=1, floor=gates[2])
        if out is not None:
            ops.gemm(out, y, self.w_o, exact=exact)
        else:
            ops.gemm(residual, y, self.w_o, add_to_out=True, exact=exact)


class ConvTail(Mixer):
    """The last taps - 1 inputs of a short convolution inside a mixer: a second piece of state per request beside the mixer's own."""
    capturable = True

    def __init__(self, keep: int, width: int, dtype, rt):
        self.keep, self.width, self.dtype, self.rt, self.spec = keep, width, dtype, rt, None

    def state_need(self):
        return StateNeed((self.keep, self.width), self.dtype) if self.keep > 0 else None


class StateSpace(RecurrentMixer):
    """params: prefix, hidden, heads, value_dim (a head's channels), state (N), groups, taps, norm_parts, eps. Tensors: prefix + in
    [2 * heads * value_dim + 2 * groups * state + heads, hidden], conv [heads * value_dim + 2 * groups * state, taps], conv.b, dt_bias, A_log, D [heads],
    norm [heads * value_dim], o."""

    @classmethod
    def tensors(cls, spec):
        p = spec.params
        pre, h, H, dv, N, G = p["prefix"], p["hidden"], p["heads"], p["value_dim"], p["state"], p["groups"]
        inner, conv = H * dv, H * dv + 2 * G * N
        return {pre + "in": TensorRule((2 * inner + 2 * G * N + H, h), "fan_in"), pre + "conv": TensorRule((conv, p["taps"]), "filter"),
                pre + "conv.b": TensorRule((conv,), "bias"), pre + "dt_bias": TensorRule((H,), "bias"), pre + "A_log": TensorRule((H,), "log_rate"),
                pre + "D": TensorRule((H,), "norm"), pre + "norm": TensorRule((inner,), "norm"), pre + "o": TensorRule((h, inner), "fan_in")}

    def __init__(self, spec, weights, rt):
        p = spec.params
        super().__init__(PartSpec(spec.kind, {**p, "key_dim": p["state"]}), weights, rt)
        self.spec = spec
        pre = p["prefix"]
        self.groups, self.taps, self.norm_parts = int(p["groups"]), int(p["taps"]), int(p["norm_parts"])
        self.inner = self.heads * self.dv
        self.conv_width = self.inner + 2 * self.groups * self.dk
        if self.groups <= 0 or self.heads % self.groups or self.norm_parts <= 0 or self.inner % self.norm_parts or not 1 <= self.taps <= ops.CONV_MAX_TAPS:
            raise AlofaError("invalid_argument", "groups divide the heads, the norm's parts divide the row, and the convolution has 1 to 16 taps",
                             f"heads={self.heads} groups={self.groups} norm_parts={self.norm_parts} taps={self.taps}")
        w_in = weights[pre + "in"]
        if w_in.shape[0] % 8:      # (rows of the projection stay 16-byte aligned)
            w_in = torch.cat([w_in, torch.zeros((8 - w_in.shape[0] % 8, w_in.shape[1]), dtype=w_in.dtype, device=w_in.device)])
        self.w_in, self.w_o = rt.matrix(w_in), rt.matrix(weights[pre + "o"])
        self.conv_w, self.conv_b = rt.vector(weights[pre + "conv"]), rt.vector(weights[pre + "conv.b"])
        self.dt_bias, self.a_log, self.skip = rt.vector(weights[pre + "dt_bias"]), rt.vector(weights[pre + "A_log"]), rt.vector(weights[pre + "D"])
        self.norm = rt.vector(weights[pre + "norm"])
        self.tail = ConvTail(self.taps - 1, self.conv_width, rt.dtype, rt)

    def stateful_parts(self):
        return [self, self.tail]

    def forward(self, ctx, where, x, residual, out=None):
        T, H, N, dv, inner = x.shape[0], self.heads, self.dk, self.dv, self.inner
        entry, k = where if isinstance(where, tuple) else (where, 0)
        exact, rows = self.rt.exact, rows_of_requests(ctx)
        proj = ctx.scratch("recurrent_proj", (T, self.w_in.shape[0]), self.rt.dtype)
        ops.gemm(proj, x, self.w_in, exact=exact)
        z, raw, dt = proj[:, :inner], proj[:, inner:inner + self.conv_width], proj[:, inner + self.conv_width:inner + self.conv_width + H]
        xbc = ctx.scratch("state_space_conv", (T, self.conv_width), self.rt.dtype)
        qf, kf = ctx.scratch("memory_q", (T, H * N), torch.float32), ctx.scratch("memory_k", (T, H * N), torch.float32)
        vf, decay = ctx.scratch("memory_v", (T, inner), torch.float32), ctx.scratch("recurrent_decay", (T, H * N), torch.float32)
        tail = ctx.state((entry, k + 1)) if self.taps > 1 else None
        if rows.offsets is None:      # single rows (decoding): the convolution and its state's step are one launch
            ops.ssd_step(xbc, raw, self.conv_w, self.conv_b, tail, rows, qf, kf, vf, decay, dt, self.dt_bias, self.a_log, H, self.groups, N, dv, exact)
        else:
            if tail is not None:
                ops.conv_bias_act(xbc, raw, self.conv_w, self.conv_b, tail, rows, silu=True, exact=exact)
                ops.conv_keep(tail, raw, rows)
            else:
                none = ctx.scratch("conv_no_state", (ctx.fn.cache.max_requests, 0, self.conv_width), self.rt.dtype)
                ops.conv_bias_act(xbc, raw, self.conv_w, self.conv_b, none, rows, silu=True, exact=exact)
            ops.ssd_operands(qf, kf, vf, decay, xbc, dt, self.dt_bias, self.a_log, H, self.groups, N, dv, exact)
        o = self._readouts(ctx, T)
        parts = ops.linear_recurrence(o, qf, kf, vf, ctx.state((entry, k)), rows, H, N, dv, ops.DECAY_GIVEN, decay)
        y = ctx.scratch("recurrent_gated", (T, inner), self.rt.dtype)
        ops.ssd_finish(y, o, xbc[:, :inner], z, self.skip, self.norm, H, dv, self.norm_parts, self.eps, exact, parts=parts)
        if out is not None:
            ops.gemm(out, y, self.w_o, exact=exact)
        else:
            ops.gemm(residual, y, self.w_o, add_to_out=True, exact=exact)


MIXES = ("r", "k", "v", "g", "w")


class TokenShift(TimeConv):
    """out[s] = x + (x' - x) * mu_s for every mix s, x' the row before (zeros before a request's first token); the last
    row is the part's state per request. params: names (the mu tensors, one per mix), width."""
    capturable = True

    @classmethod
    def tensors(cls, spec):
        return {n: TensorRule((spec.params["width"],), "unit_interval") for n in spec.params["names"]}

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        self.width = int(spec.params["width"])
        self.mu = rt.vector(torch.stack([weights[n].float() for n in spec.params["names"]]))

    def state_need(self):
        return StateNeed((1, self.width), self.rt.dtype)

    def forward(self, ctx, where, out, x):
        state, rows = ctx.state(where), rows_of_requests(ctx)
        single = rows.offsets is None      # single rows (decoding): the mix and the state's step are one launch
        ops.shift_mix(out, x, self.mu, state, rows, keep=single)
        if not single:
            ops.keep_last_rows(state, x, rows)


class TimeMix(RecurrentMixer):
    """params: prefix, hidden, heads, key_dim (value heads have the same size), rank (of the decay's two-step
    projection), eps. Tensors: prefix + mu.r/k/v/g/w, r, k, v, g, o, w1 [rank, hidden], w2 [heads * key_dim, rank], w0,
    u [heads, key_dim], norm [heads * key_dim]."""

    @classmethod
    def shift_spec(cls, spec) -> PartSpec:
        return PartSpec("token_shift", {"names": tuple(spec.params["prefix"] + "mu." + s for s in MIXES), "width": spec.params["hidden"]})

    @classmethod
    def tensors(cls, spec):
        p = spec.params
        pre, h, kd, r = p["prefix"], p["hidden"], p["heads"] * p["key_dim"], p["rank"]
        out = dict(TokenShift.tensors(cls.shift_spec(spec)))
        out.update({pre + n: TensorRule((kd, h), "fan_in") for n in ("r", "k", "v", "g")})
        out.update({pre + "w1": TensorRule((r, h), "fan_in"), pre + "w2": TensorRule((kd, r), "fan_in"), pre + "w0": TensorRule((kd,), "log_rate"),
                    pre + "u": TensorRule((p["heads"], p["key_dim"]), "bias"), pre + "norm": TensorRule((kd,), "norm"), pre + "o": TensorRule((h, kd), "fan_in")})
        return out

    def __init__(self, spec, weights, rt):
        if spec.params.get("value_dim") not in (None, spec.params["key_dim"]):
            raise AlofaError("invalid_argument", "time mixing has value heads of the key heads' size", f"key_dim={spec.params['key_dim']} value_dim={spec.params['value_dim']}")
        super().__init__(spec, weights, rt)
        p, pre = spec.params, spec.params["prefix"]
        self.rank = int(p["rank"])
        self.shift = build_part("conv", self.shift_spec(spec), weights, rt)
        self.w = {n: rt.matrix(weights[pre + n]) for n in ("r", "k", "v", "g", "w1", "w2", "o")}
        self.w_o = self.w["o"]
        self.w0, self.norm = rt.vector(weights[pre + "w0"]), rt.vector(weights[pre + "norm"])
        self.bonus = rt.vector(weights[pre + "u"])

    def stateful_parts(self):
        return [self, self.shift]

    def forward(self, ctx, where, x, residual, out=None):
        T, kd = x.shape[0], self.heads * self.dk
        entry, k = where if isinstance(where, tuple) else (where, 0)
        exact = self.rt.exact
        mixes = ctx.scratch("time_mix_inputs", (len(MIXES), T, self.hidden), self.rt.dtype)
        self.shift.forward(ctx, (entry, k + 1), mixes, x)
        proj = ctx.scratch("time_mix_proj", (T, 4 * kd), self.rt.dtype)
        for i, n in enumerate(("r", "k", "v", "g")):
            ops.gemm(proj[:, i * kd:(i + 1) * kd], mixes[i], self.w[n], exact=exact)
        low = ctx.scratch("time_mix_low", (T, self.rank), self.rt.dtype)
        ops.gemm(low, mixes[4], self.w["w1"], exact=exact)
        ops.activation(low, low, ops.TANH, exact=exact)
        z = ctx.scratch("recurrent_decay", (T, kd), torch.float32)
        ops.gemm(z, low, self.w["w2"], self.w0, exact=exact)
        o = self._readouts(ctx, T)
        parts = ops.linear_recurrence(o, proj[:, :kd], proj[:, kd:2 * kd], proj[:, 2 * kd:3 * kd], ctx.state((entry, k)), rows_of_requests(ctx),
                                      self.heads, self.dk, self.dv, ops.DECAY_EXP_NEG_EXP, z, bonus=self.bonus, before_update=True)
        self._leave(ctx, o, parts, proj[:, 3 * kd:], self.norm, residual, out)


class ParallelMixers(Mixer):
    """Several mixers side by side that read the same rows; the result is the sum of theirs, each times its scale.
    params: branches (PartSpecs of mixers that take ``out=``), scales (one per branch), hidden; norms (optional: one tensor name per
    branch, a weight [hidden] each: every branch's result passes an RMS norm over the width with that weight before the sum; two
    branches) and eps."""

    @classmethod
    def tensors(cls, spec):
        from .base import tensors_of
        out = {}
        for b in spec.params["branches"]:
            out.update(tensors_of("mixer", b))
        for name in spec.params.get("norms") or ():
            out[name] = TensorRule((spec.params["hidden"],), "norm")
        return out

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        p = spec.params
        self.hidden = int(p["hidden"])
        self.branches = [build_part("mixer", b, weights, rt) for b in p["branches"]]
        self.scales = [float(s) for s in p["scales"]]
        if not self.branches or len(self.scales) != len(self.branches):
            raise AlofaError("invalid_argument", "one scale per branch, and at least one branch", f"branches={len(self.branches)} scales={len(self.scales)}")
        self.norms = [rt.vector(weights[n]) for n in p.get("norms") or ()]
        self.eps = float(p.get("eps", 1e-6))
        if self.norms and (len(self.norms) != 2 or len(self.branches) != 2):
            raise AlofaError("unsupported", "branches that are normed before the sum come in pairs, a norm each", f"branches={len(self.branches)} norms={len(self.norms)}")

    @property
    def capturable(self):
        return all(b.capturable for b in self.branches)

    def stateful_parts(self):
        return [part for b in self.branches for part in b.stateful_parts()]

    def prepare(self, n_positions):
        for b in self.branches:
            b.prepare(n_positions)

    @property
    def takes_channel_scale(self):
        """Normed branches join the stream in a launch of their own, which also applies a factor per channel (``scale=``) and leaves the next norm (``then=``)."""
        return bool(self.norms)

    def forward(self, ctx, where, x, residual, out=None, scale=None, then=None):
        entry, k = where if isinstance(where, tuple) else (where, 0)
        outs = []
        for j, b in enumerate(self.branches):
            buf = ctx.scratch(f"branch_{j}", tuple(residual.shape), torch.float32)
            b.forward(ctx, (entry, k), x, residual, out=buf)
            k += len(b.stateful_parts())
            outs.append(buf)
        if self.norms:
            if out is not None:
                ops.rms_pair_sum(out, outs[0], self.norms[0], self.scales[0], outs[1], self.norms[1], self.scales[1], self.eps, self.rt.exact)
            else:
                ops.rms_pair_add_norm(residual, outs[0], self.norms[0], self.scales[0], outs[1], self.norms[1], self.scales[1], scale, self.eps, self.rt.exact, then_norm=then)
            return
        target = residual
        if out is not None:
            out.zero_()
            target = out
        for j in range(0, len(outs), 2):
            pair = outs[j:j + 2]
            ops.add_scaled(target, pair[0], self.scales[j], pair[1] if len(pair) > 1 else None, self.scales[j + 1] if len(pair) > 1 else 0.0, self.rt.exact)


register_part("mixer", "retention", Retention)
register_part("mixer", "gated_linear", GatedLinearAttention)
register_part("mixer", "time_mix", TimeMix)
register_part("mixer", "lightning_attention", LightningAttention)
register_part("mixer", "matrix_memory", MatrixMemory)
register_part("mixer", "state_space", StateSpace)
register_part("mixer", "parallel", ParallelMixers)
register_part("conv", "token_shift", TokenShift)

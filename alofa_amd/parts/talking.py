"""Attention whose heads talk after the softmax, with values that carry their positions.

q = Wq x, k = Wk x, v = Wv x (heads side by side, query/key heads of ``head_dim`` and value heads of ``v_head_dim`` channels). Queries
and keys take the position encoding on their first channels and are then (``unit_norm``) divided by their root mean square; values
(``value_position``) are turned by their own positions on all channels and kept so. Per query head g the softmax of scale * q_g . k over
the keys a row may see (all before it, or the last ``window``); then the heads' weights are mixed, w_h = sum_g M[h, g] p_g (``talk``), and
head h applies w_h to the values of its own key/value head; what comes out is turned back by the row's own position, multiplied by
sigmoid(Wg x) (``gate``), and projected by Wo.

A layer may have no key and value projections of its own and read the pages of an earlier layer (``owns_cache`` False; its run entry
names that layer with ``cache_of``): it brings its own queries, window, mixing matrix and gate.

The pages hold keys as [kv_head, slot, head_dim] and values transposed, [kv_head, v_head_dim, slot], as the other attention parts'
(``keep_window``: how long they are kept: the longest window among the layers that read them).

Mixing the weights is linear in what they are applied to: head h's result is sum_g M[h, g] A[c(h)][g], where A[c][g] are query head g's
unmixed weights applied to the values of value head c. In bfloat16, with pages of a power of two and heads of one size that the
matrix-core attention kernels are built for, those kernels serve every value head in turn within one launch (portions of prompts through
the prefill kernel, single tokens through the decode kernel, as in ``paged_attend``) and leave A unrounded; one small kernel then mixes, turns back and
gates. The softmax weights are 32-bit numbers in this part: they meet the values as two bfloat16 numbers each, the rounding and what it
took away (``fine_weights``), so that sixteen bits of every weight count. Every other case (float32, other sizes) runs the always-valid kernel, a block per row."""
from __future__ import annotations

import torch

from .. import ops
from ..errors import AlofaError
from ..weights.loader import TensorRule
from .attention import RowPlan
from .base import SLOT, CacheNeed, CacheTensor, Mixer, build_part, register_part

NAMES = {"q": "q", "k": "k", "v": "v", "o": "o", "gate": "g", "talk": "talk"}


class TalkingAttention(Mixer):
    """params: prefix, hidden, heads, kv_heads, head_dim, v_head_dim, scale, window (None or a count of keys), keep_window (None: every
    key is kept; default ``window``), position (PartSpec of a rotary encoding whose head_dim is the count of turned channels),
    value_position (the same for value heads, or None), unit_norm, eps, talk (bool), gate (bool), owns_cache (bool), names, init."""
    capturable = True

    @classmethod
    def tensors(cls, spec):
        p = spec.params
        n, init = {**NAMES, **p.get("names", {})}, p.get("init", "fan_in")
        pre, h, H, G, d, dv = p["prefix"], p["hidden"], p["heads"], p["kv_heads"], p["head_dim"], p["v_head_dim"]
        out = {pre + n["q"]: TensorRule((H * d, h), init)}
        if p.get("owns_cache", True):
            out.update({pre + n["k"]: TensorRule((G * d, h), init), pre + n["v"]: TensorRule((G * dv, h), init)})
        if p.get("talk", False):
            out[pre + n["talk"]] = TensorRule((H, H), "head_mix")
        if p.get("gate", False):
            out[pre + n["gate"]] = TensorRule((H * dv, h), init)
        out[pre + n["o"]] = TensorRule((h, H * dv), init)
        return out

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        p = spec.params
        self.hidden, self.heads, self.kv_heads = int(p["hidden"]), int(p["heads"]), int(p["kv_heads"])
        self.d, self.dv = int(p["head_dim"]), int(p["v_head_dim"])
        self.window = p.get("window")
        self.keep_window = p["keep_window"] if "keep_window" in p else self.window
        self.owns = bool(p.get("owns_cache", True))
        self.scale, self.eps, self.unit_norm = float(p["scale"]), float(p.get("eps", 1e-6)), bool(p.get("unit_norm", False))
        if self.kv_heads <= 0 or self.heads % self.kv_heads:
            raise AlofaError("unsupported", "kv_heads must be positive and divide heads", f"heads={self.heads} kv_heads={self.kv_heads}")
        if not 0 < self.d <= ops.MAX_HEAD_DIM or not 0 < self.dv <= ops.MAX_HEAD_DIM or self.dv % 2:
            raise AlofaError("unsupported", f"heads of up to {ops.MAX_HEAD_DIM} channels; an even value size", f"head_dim={self.d} v_head_dim={self.dv}")
        if self.window is not None and self.window <= 0:
            raise AlofaError("invalid_argument", "an attention window must be positive", f"window={self.window}")
        if self.keep_window is not None and (self.window is None or self.keep_window < self.window):
            raise AlofaError("invalid_argument", "keys are kept at least as long as this layer sees them", f"window={self.window} keep_window={self.keep_window}")
        pre, n = p["prefix"], {**NAMES, **p.get("names", {})}
        self.position = build_part("position", p["position"], weights, rt)
        self.value_position = build_part("position", p["value_position"], weights, rt) if p.get("value_position") is not None else None
        if self.position.head_dim > self.d or (self.value_position is not None and self.value_position.head_dim != self.dv):
            raise AlofaError("invalid_argument", "turned channels: at most a head's, and all of a value head's", f"head_dim={self.d} v_head_dim={self.dv}")
        mats = [weights[pre + n["q"]]] + ([weights[pre + n["k"]], weights[pre + n["v"]]] if self.owns else [])
        self.gate_at = sum(m.shape[0] for m in mats)
        self.gated = bool(p.get("gate", False))
        if self.gated:
            mats.append(weights[pre + n["gate"]])
        if len({m.dtype for m in mats}) > 1:
            mats = [m.float() for m in mats]
        self.w_in = rt.matrix(torch.cat(mats, dim=0))
        self.w_o = rt.matrix(weights[pre + n["o"]])
        self.talk = rt.vector(weights[pre + n["talk"]]) if p.get("talk", False) else None
        self.q_width = self.heads * self.d
        self.qkv_width = self.q_width + (self.kv_heads * (self.d + self.dv) if self.owns else 0)

    def cache_need(self):
        return CacheNeed((CacheTensor("k", (self.kv_heads, SLOT, self.d)), CacheTensor("v", (self.kv_heads, self.dv, SLOT))), self.keep_window)

    def prepare(self, n_positions):
        self.position.table(n_positions)
        if self.value_position is not None:
            self.value_position.table(n_positions)

    def _on_matrix_cores(self, ctx, kc, proj) -> bool:
        page = kc.shape[2]
        plan = ctx.memo("gqa_attention.rows", lambda: RowPlan(ctx))
        return (not self.rt.exact and self.rt.dtype is torch.bfloat16 and self.d == self.dv and self.d % 16 == 0
                and page >= ops.MIN_FAST_PAGE and page & (page - 1) == 0 and proj.stride(0) % 8 == 0 and (self.heads * self.dv) % 4 == 0
                and (plan.long_runs is None or self.d in ops.PREFILL_HEAD_DIMS))

    def _attend_per_value_head(self, ctx, q, kc, vc, table, attn, v_table, gate) -> None:
        T = q.shape[0]
        plan = ctx.memo("gqa_attention.rows", lambda: RowPlan(ctx))
        applied = ctx.scratch("talking_applied", (self.kv_heads, T, self.heads * self.dv), torch.float32)
        common = (self.heads, self.kv_heads, self.d, self.window, self.scale)
        if plan.long_runs is not None:
            tiles, share, rows = plan.tiles(self.heads, self.kv_heads, self.d, self.window, plain=True)
            ops.attention_prefill(applied, q, kc, vc, table, tiles, *common, share=share, rows=rows, fine_weights=True, all_value_heads=True)
        if plan.n_short:
            # (one launch for all value heads: its grid, its parts and its scratch count (token, value head) pairs)
            floats = ops.decode_scratch_floats(plan.n_short * self.kv_heads, self.heads, self.kv_heads, self.d, ctx.max_context, self.window)
            partial = ctx.scratch("attn_partial", (floats,), torch.float32) if floats else None
            one_each = ctx.max_q_len == 1 and plan.short_rows is None and plan.long_runs is None
            ops.attention_decode(applied, q, kc, vc, table, None if one_each else ctx.req_of_token, ctx.positions, *common,
                                 ctx.max_context, partial, rows=plan.short_rows, fine_weights=True, all_value_heads=True)
        ops.talk_mix(attn, applied, ctx.positions, self.heads, self.kv_heads, self.dv, self.talk, v_table, gate)

    def forward(self, ctx, where, x, residual, out=None):
        T, exact = residual.shape[0], self.rt.exact
        kv = ctx.kv(where)
        if kv.owner != self.owns:
            raise AlofaError("invalid_argument", "a layer with key and value projections owns its pages, one without reads another's", f"where={where} owns={self.owns}")
        proj = ctx.scratch("talking_proj", (T, self.w_in.shape[0]), self.rt.dtype)
        ops.gemm(proj, x, self.w_in, exact=exact)
        v_table = self.value_position.table(ctx.n_positions) if self.value_position is not None else None
        kc, vc = kv.tensors["k"], kv.tensors["v"]
        ops.turn_norm_write(proj[:, :self.qkv_width], ctx.positions, self.position.table(ctx.n_positions), v_table, self.heads,
                            self.kv_heads if self.owns else 0, self.d, self.dv, self.eps, self.unit_norm, exact,
                            kv.slots if self.owns else None, kc if self.owns else None, vc if self.owns else None)
        attn = ctx.scratch("talking_out", (T, self.heads * self.dv), self.rt.dtype)
        gate = proj[:, self.gate_at:] if self.gated else None
        if self._on_matrix_cores(ctx, kc, proj):
            self._attend_per_value_head(ctx, proj[:, :self.q_width], kc, vc, kv.block_table, attn, v_table, gate)
        else:
            ops.talking_attention(attn, proj[:, :self.q_width], kc, vc, kv.block_table, ctx.req_of_token, ctx.positions, self.heads, self.kv_heads,
                                  self.d, self.dv, self.window, self.scale, self.talk, v_table, gate, exact)
        if out is not None:
            ops.gemm(out, attn, self.w_o, exact=exact)
        else:
            ops.gemm(residual, attn, self.w_o, add_to_out=True, exact=exact)


register_part("mixer", "talking_attention", TalkingAttention)

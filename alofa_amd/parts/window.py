"""Softmax attention over a window of a paged cache, with what some designs add to it.

q = Wq x, k = Wk x, v = Wv x (``heads`` query heads and ``kv_heads`` key/value heads of ``head_dim`` and ``v_head_dim`` channels; query head h
reads key/value head h // (heads / kv_heads)). Then, each optional and chosen by a parameter:

  qk_norm     queries and keys are divided by a root mean square and multiplied by a weight before they are turned: "head" (every head by its
              own, one weight vector [head_dim] for all heads), "all" (the whole query projection of a row by one root mean square, and the whole
              key projection by another; weights [heads * head_dim] and [kv_heads * head_dim]), "unit" (every head by its own, no weight).
  position    a position encoding with a table (``rotary`` in any of its forms), or None.
  values_are_keys   there is no Wv: a token's value is its key as projected, before norm and turn.
  window      row i sees the tokens j with 0 <= i - j < window.
  pool        P: beside the window's tokens, one key and one value for every block of P tokens that lies wholly behind the window (block b holds
              the tokens b P .. b P + P - 1 and is seen when b P + P - 1 <= i - window): the means of the block's keys and values as the pages
              hold them. Tokens that have left the window and whose block is not yet whole behind it are not seen. One softmax over both.
  bias        a learned bias by distance, added to the scaled score: table[bucket(i - j), h] with ``rows`` rows: bucket(n) = n below rows/2, else
              min(rows - 1, rows/2 + floor(ln(n / (rows/2)) / ln(far / (rows/2)) * (rows - rows/2))).
  sink        a number per head whose exponential joins the softmax's denominator (no key, no value).
  gate        "channel": the heads' outputs times sigmoid(Wg x), one gate per output channel; "head": one gate per head.

Then the output projection. Scores, the softmax, norms and angles are float32 (float64 sums in the exact path); on the matrix cores every
softmax weight meets the values as two bfloat16 numbers, its rounding and what the rounding took away.

The pages hold keys as [kv_head, slot, d] and values transposed, [kv_head, d, slot], as the other attention parts' (heads of unequal key and
value size are widened with zero rows to one size d, so that the matrix-core kernels can read them). The pooled blocks live in pages of their own
(``PooledBlocks``, a second stateful part of the mixer) that are never given back while the request lives: one place per P tokens of a page."""
from __future__ import annotations

import math
import os

import torch

from .. import ops
from ..errors import AlofaError
from ..weights.loader import TensorRule
from .attention import GQAAttention, RowPlan, _padded_heads
from .base import SLOT, CacheNeed, CacheTensor, Mixer, build_part, part_class, register_part

NAMES = {"q": "q", "k": "k", "v": "v", "o": "o", "gate": "g", "q_norm": "q.norm", "k_norm": "k.norm", "bias": "rel", "sink": "sink"}


USE_SPAN_MFMA = os.environ.get("ALOFA_SPAN_MFMA", "1") != "0"      # 0 (for measurements): pooled blocks, bias and sink go through the always-valid kernel in bfloat16 too


def _runs_of_sixteen(ctx) -> torch.Tensor:
    """The step's rows as runs of up to sixteen rows of one request: int32 [n, 3] (request index, first row, rows)."""
    runs = [(i, s.row0 + q0, min(16, s.n - q0)) for i, s in enumerate(ctx.spans) for q0 in range(0, s.n, 16)]
    return torch.tensor(runs, dtype=torch.int32, device=ctx.device)


def distance_buckets(rows: int, far: float, upto: int) -> list:
    """The bias table's row for every distance 0 .. upto - 1."""
    half = rows // 2
    out = []
    for n in range(upto):
        if n < half:
            out.append(n)
        else:
            out.append(min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (rows - half)))))
    return out


class PooledBlocks(Mixer):
    """The pages of the pooled blocks of a ``window_attention``: mean keys and mean values, one place per ``pool`` tokens, kept for good."""
    capturable = True

    def __init__(self, kv_heads: int, d: int, pool: int, rt):
        self.kv_heads, self.d, self.pool, self.rt, self.spec = kv_heads, d, pool, rt, None

    def cache_need(self):
        return CacheNeed((CacheTensor("pk", (self.kv_heads, SLOT, self.d), every=self.pool), CacheTensor("pv", (self.kv_heads, self.d, SLOT), every=self.pool)), None)


class WindowAttention(Mixer):
    """params: prefix, hidden, heads, kv_heads, head_dim, v_head_dim, scale, window, position (PartSpec or None), qk_norm (None, "head", "all", "unit"), eps,
    values_are_keys, pool (None or P), bias (None or {"rows": n, "far": D}), sink (bool), gate (None, "channel", "head"), names, init."""
    capturable = True

    @classmethod
    def tensors(cls, spec):
        p = spec.params
        n, init = {**NAMES, **p.get("names", {})}, p.get("init", "fan_in")
        pre, h, H, G, d = p["prefix"], p["hidden"], p["heads"], p["kv_heads"], p["head_dim"]
        dv = d if p.get("values_are_keys", False) else (p.get("v_head_dim") or d)
        out = {pre + n["q"]: TensorRule((H * d, h), init), pre + n["k"]: TensorRule((G * d, h), init)}
        if not p.get("values_are_keys", False):
            out[pre + n["v"]] = TensorRule((G * dv, h), init)
        if p.get("qk_norm") == "head":
            out.update({pre + n["q_norm"]: TensorRule((d,), "norm"), pre + n["k_norm"]: TensorRule((d,), "norm")})
        elif p.get("qk_norm") == "all":
            out.update({pre + n["q_norm"]: TensorRule((H * d,), "norm"), pre + n["k_norm"]: TensorRule((G * d,), "norm")})
        if p.get("bias") is not None:
            out[pre + n["bias"]] = TensorRule((p["bias"]["rows"], H), "unit")
        if p.get("sink", False):
            out[pre + n["sink"]] = TensorRule((H,), "unit")
        if p.get("gate") == "channel":
            out[pre + n["gate"]] = TensorRule((H * dv, h), init)
        elif p.get("gate") == "head":
            out[pre + n["gate"]] = TensorRule((H, h), init)
        out[pre + n["o"]] = TensorRule((h, H * dv), init)
        return out

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        p = spec.params
        self.hidden, self.heads, self.kv_heads = int(p["hidden"]), int(p["heads"]), int(p["kv_heads"])
        self.values_are_keys = bool(p.get("values_are_keys", False))
        self.qk_dim = int(p["head_dim"])
        self.v_dim = self.qk_dim if self.values_are_keys else int(p.get("v_head_dim") or self.qk_dim)
        self.d = GQAAttention.common_head_size(self.qk_dim, self.v_dim)      # (one size for keys and values in the pages)
        self.window, self.pool = p.get("window"), p.get("pool")
        self.scale, self.eps = float(p["scale"]), float(p.get("eps", 1e-6))
        self.norm_kind, self.gate_kind = p.get("qk_norm"), p.get("gate")
        if self.kv_heads <= 0 or self.heads % self.kv_heads:
            raise AlofaError("unsupported", "kv_heads must be positive and divide heads", f"heads={self.heads} kv_heads={self.kv_heads}")
        if self.d % 2 or not 2 <= self.d <= ops.MAX_HEAD_DIM:
            raise AlofaError("unsupported", f"the attention kernels take even head sizes up to {ops.MAX_HEAD_DIM}", f"head_dim={self.d}")
        if self.window is not None and self.window <= 0:
            raise AlofaError("invalid_argument", "an attention window must be positive", f"window={self.window}")
        if self.pool is not None and (self.window is None or self.pool <= 0):
            raise AlofaError("invalid_argument", "pooled blocks of a positive size lie behind a window", f"window={self.window} pool={self.pool}")
        if self.norm_kind not in (None, "head", "all", "unit") or self.gate_kind not in (None, "channel", "head"):
            raise AlofaError("unsupported", "no such norm of queries and keys, or no such gate", f"qk_norm={self.norm_kind} gate={self.gate_kind}")
        pre, n = p["prefix"], {**NAMES, **p.get("names", {})}
        H, G, D = self.heads, self.kv_heads, self.d
        order = None
        self.position = None
        if p.get("position") is not None:
            position = p["position"]
            if D != self.qk_dim:
                position = part_class("position", position.kind).for_head(position, D)
            self.position = build_part("position", position, weights, rt)
            if self.position.table(1) is None:
                raise AlofaError("unsupported", "this mixer takes position encodings that give a table of angles", f"position={position.kind}")
            order = self.position.channel_order()
        mats = [_padded_heads(weights[pre + n["q"]], H, self.qk_dim, D, order), _padded_heads(weights[pre + n["k"]], G, self.qk_dim, D, order)]
        if not self.values_are_keys:
            mats.append(_padded_heads(weights[pre + n["v"]], G, self.v_dim, D))
        self.qkv_width = sum(m.shape[0] for m in mats)
        self.gate_width = 0
        if self.gate_kind is not None:
            mats.append(weights[pre + n["gate"]])
            self.gate_width = mats[-1].shape[0]
        rows = self.qkv_width + self.gate_width
        if rows % 8:      # (rows of the projection stay 16-byte aligned)
            mats.append(torch.zeros((8 - rows % 8, self.hidden), dtype=mats[0].dtype, device=mats[0].device))
        if len({m.dtype for m in mats}) > 1:
            mats = [m.float() for m in mats]
        self.w_in = rt.matrix(torch.cat(mats, dim=0))
        w_o = weights[pre + n["o"]]
        if D != self.v_dim:      # zero columns where the value heads were widened
            w_o = _padded_heads(w_o.t(), H, self.v_dim, D).t()
        self.w_o = rt.matrix(w_o)
        self.scope, self.wq, self.wk = ops.NORM_NONE, None, None
        if self.norm_kind == "unit":
            self.scope = ops.NORM_HEAD
        elif self.norm_kind == "head":
            self.scope = ops.NORM_HEAD
            self.wq = rt.vector(_padded_heads(weights[pre + n["q_norm"]].float(), 1, self.qk_dim, D, order))
            self.wk = rt.vector(_padded_heads(weights[pre + n["k_norm"]].float(), 1, self.qk_dim, D, order))
        elif self.norm_kind == "all":
            self.scope = ops.NORM_ALL
            self.wq = rt.vector(_padded_heads(weights[pre + n["q_norm"]].float(), H, self.qk_dim, D, order))
            self.wk = rt.vector(_padded_heads(weights[pre + n["k_norm"]].float(), G, self.qk_dim, D, order))
        self.bias = None
        if p.get("bias") is not None:
            table = weights[pre + n["bias"]].float()                 # [rows, heads]
            rows_n, far = int(p["bias"]["rows"]), float(p["bias"]["far"])
            if table.shape[0] != rows_n or rows_n < 2 or not far > rows_n // 2:
                raise AlofaError("invalid_argument", "the bias table has at least two rows and reaches beyond its evenly spaced half", f"rows={rows_n} far={far}")
            # every distance the window lets through has its row; beyond ``far`` all distances share the last one
            upto = int(math.ceil(far)) + 1 if self.window is None else min(int(self.window), int(math.ceil(far)) + 1)
            self.bias = rt.vector(table[torch.tensor(distance_buckets(rows_n, far, upto), device=table.device)].t().contiguous())      # [heads, distances]
        self.sink = rt.vector(weights[pre + n["sink"]]) if p.get("sink", False) else None
        self.pooled = PooledBlocks(G, D, int(self.pool), rt) if self.pool is not None else None
        # the pages are kept as long as a block that a row completes can still be read whole
        self.keep_window = None if self.window is None else max(int(self.window), int(self.pool or 0))

    def cache_need(self):
        return CacheNeed.keys_and_values(self.kv_heads, self.d, self.keep_window)

    def stateful_parts(self):
        return [self] if self.pooled is None else [self, self.pooled]

    def prepare(self, n_positions):
        if self.position is not None:
            self.position.table(n_positions)

    def _plain_on_matrix_cores(self, ctx, kc) -> bool:
        page = kc.shape[2]
        if self.pooled is not None or self.bias is not None or self.sink is not None or self.rt.exact or self.rt.dtype is not torch.bfloat16:
            return False
        plan = ctx.memo("gqa_attention.rows", lambda: RowPlan(ctx))
        return self.d % 16 == 0 and page >= ops.MIN_FAST_PAGE and page & (page - 1) == 0 and (plan.long_runs is None or self.d in ops.PREFILL_HEAD_DIMS)

    def _attend_plain(self, ctx, q, kv, attn) -> None:
        plan = ctx.memo("gqa_attention.rows", lambda: RowPlan(ctx))
        common = (self.heads, self.kv_heads, self.d, self.window, self.scale)
        if plan.long_runs is not None:
            # (softmax weights are 32-bit numbers in this part: the form of the kernel that takes them as two bfloat16 numbers each)
            tiles, share, rows = plan.tiles(self.heads, self.kv_heads, self.d, self.window, plain=True)
            ops.attention_prefill(attn, q, kv.k, kv.v, kv.block_table, tiles, *common, share=share, rows=rows, fine_weights=True)
        if plan.n_short:
            floats = ops.decode_scratch_floats(plan.n_short, self.heads, self.kv_heads, self.d, ctx.max_context, self.window)
            partial = ctx.scratch("attn_partial", (floats,), torch.float32) if floats else None
            one_each = ctx.max_q_len == 1 and plan.short_rows is None and plan.long_runs is None
            ops.attention_decode(attn, q, kv.k, kv.v, kv.block_table, None if one_each else ctx.req_of_token, ctx.positions, *common,
                                 ctx.max_context, partial, rows=plan.short_rows, fine_weights=True)

    def forward(self, ctx, where, x, residual, out=None):
        T, exact = residual.shape[0], self.rt.exact
        entry, k = where if isinstance(where, tuple) else (where, 0)
        kv = ctx.kv((entry, k))
        H, G, D = self.heads, self.kv_heads, self.d
        proj = ctx.scratch("window_proj", (T, self.w_in.shape[0]), self.rt.dtype)
        ops.gemm(proj, x, self.w_in, exact=exact)
        table = self.position.table(ctx.n_positions) if self.position is not None else None
        factors = ctx.scratch("window_row_factors", (T, 2), torch.float64) if self.scope == ops.NORM_ALL else None
        # (the norms average over the channels the design has: the widened ones are zeros and are not counted)
        ops.norm_turn_write(proj[:, :self.qkv_width], ctx.positions, table, H, G, D, D, self.scope, self.wq, self.wk, self.eps, exact, kv.slots, kv.k, kv.v,
                            self.values_are_keys, factors, true_d=self.qk_dim)
        pooled = None
        if self.pooled is not None:
            pages = ctx.kv((entry, k + 1))
            pooled = (pages.tensors["pk"], pages.tensors["pv"], pages.block_table, int(self.pool))
            ops.pool_blocks(kv.k, kv.v, pooled[0], pooled[1], kv.block_table, pages.block_table, ctx.req_of_token, ctx.positions, G, D, D, int(self.pool), exact)
        attn = ctx.scratch("window_out", (T, H * D), self.rt.dtype)
        gate = proj[:, self.qkv_width:self.qkv_width + self.gate_width] if self.gate_kind is not None else None
        if self._plain_on_matrix_cores(ctx, kv.k):
            # a window and nothing else: the engine's matrix-core kernels, portions of prompts and single tokens each by its own
            self._attend_plain(ctx, proj[:, :H * D], kv, attn)
            if gate is not None:
                ops.head_gate(attn, gate, H, self.v_dim, self.gate_kind == "head", dv_stored=D)
        elif not exact and USE_SPAN_MFMA and ops.span_attention_fast(D, kv.k.shape[2], self.rt.dtype):
            # pooled blocks, a bias or a sink: this part's own matrix-core kernel, a wavefront per run of sixteen rows and head
            tiles = None if ctx.max_q_len == 1 else ctx.memo("window_attention.runs", lambda: _runs_of_sixteen(ctx))
            kind = ops.GATE_NONE if gate is None else (ops.GATE_CHANNEL if self.gate_kind == "channel" else ops.GATE_HEAD)
            ops.span_attention_mfma(attn, proj[:, :H * D], kv.k, kv.v, kv.block_table, tiles, ctx.req_of_token, ctx.positions, H, G, D, self.window, self.scale,
                                    pooled=pooled, bias=self.bias, sink=self.sink, gate=gate, gate_kind=kind, dv_true=self.v_dim)
        elif D != self.v_dim and gate is not None and self.gate_kind == "channel":
            # (a gate per channel of the design's value heads against outputs of widened heads: applied afterwards, head by head)
            ops.span_attention(attn, proj[:, :H * D], kv.k, kv.v, kv.block_table, ctx.req_of_token, ctx.positions, H, G, D, D, self.window, self.scale, exact,
                               pooled=pooled, bias=self.bias, sink=self.sink)
            ops.head_gate(attn, gate, H, self.v_dim, False, dv_stored=D)
        else:
            kind = ops.GATE_NONE if gate is None else (ops.GATE_CHANNEL if self.gate_kind == "channel" else ops.GATE_HEAD)
            ops.span_attention(attn, proj[:, :H * D], kv.k, kv.v, kv.block_table, ctx.req_of_token, ctx.positions, H, G, D, D, self.window, self.scale, exact,
                               pooled=pooled, bias=self.bias, sink=self.sink, gate=gate, gate_kind=kind)
        if out is not None:
            ops.gemm(out, attn, self.w_o, exact=exact)
        else:
            ops.gemm(residual, attn, self.w_o, add_to_out=True, exact=exact)


register_part("mixer", "window_attention", WindowAttention)

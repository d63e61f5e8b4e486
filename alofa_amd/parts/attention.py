"""Grouped-query attention over a paged cache.

q = x Wq^T + bq, k = x Wk^T + bk, v = x Wv^T + bv, heads packed in the channel
dimension (channel = head * d + j); q and k take the position encoding, v does
not; rotated k and v go to the token's cache slot; each query head attends the
keys of key head (head // group) causally (optionally only the last ``window``
keys), scale 1/sqrt(d); then the output projection, added to the residual
stream (src/alofa/engine/executor.mojo:715-804, src/alofa/kernels/cpu/paged.mojo:249-336).

The three input projections run as one matrix product: their matrices are
stacked by rows ([out, in] layout, nothing is transposed)."""
from __future__ import annotations

import numpy as np
import torch

from .. import ops
from ..errors import AlofaError
from ..weights.loader import TensorRule
from .base import CacheNeed, Mixer, build_part, part_class, register_part


SHORT = ops.DECODE_MAX_Q     # rows of one request up to which they are served as single tokens
TILE_ROWS = 64               # rows of one block of the prefill kernel


class RowPlan:
    """How this part's bfloat16 kernels share out the rows of one step: requests that bring at
    most ``SHORT`` rows are "short" (served key-head-wise, one token at a time, by the decode
    kernel), the others are cut into runs of up to ``TILE_ROWS`` rows for the prefill kernel.
    Built once per step from the spans and used by every attention layer."""

    def __init__(self, ctx):
        spans = ctx.spans
        self.device = ctx.device
        self.n_short = sum(s.n for s in spans if s.n <= SHORT)
        self.short_rows = None      # int32 indices of the short rows; None when every row is short (or none is)
        self.long_runs = None       # (request index, first row, rows, first position) per run; None when every row is short
        self._tiles: dict = {}
        if self.n_short < ctx.tokens:
            self.long_runs = [(i, s.row0 + q0, min(TILE_ROWS, s.n - q0), s.pos0 + q0)
                              for i, s in enumerate(spans) if s.n > SHORT for q0 in range(0, s.n, TILE_ROWS)]
            if self.n_short:
                self.short_rows = torch.tensor([r for s in spans if s.n <= SHORT for r in range(s.row0, s.row0 + s.n)],
                                               dtype=torch.int32, device=self.device)

    def tiles(self, heads: int, kv_heads: int, d: int, window, plain: bool = False):
        """The runs as blocks of the prefill kernel for a mixer with these head counts, how many heads
        of a group share a block's tiles and how many rows a wave owns (all three depend on how many
        blocks there are). ``plain``: every head has blocks of its own and a wave owns 16 rows (the
        one form of the kernel that takes the weights in two parts)."""
        key = (heads, kv_heads, d, window, plain)
        if key not in self._tiles:
            share = 0 if plain else ops.prefill_share(heads, kv_heads, d, len(self.long_runs))
            rows = 16 if plain else ops.prefill_rows(heads, kv_heads, d, share, len(self.long_runs))
            per_run = ops.prefill_blocks_per_run(heads, kv_heads, share, rows)
            self._tiles[key] = (torch.tensor(ops.pair_tiles(self.long_runs, window, per_run), dtype=torch.int32, device=self.device), share, rows)
        return self._tiles[key]


def paged_attend(ctx, entry, qkv, attn, heads, kv_heads, d, window, scale, position, rt) -> None:
    """The rows of one step through attention over the pages of the mixer at ``entry``: ``qkv`` [T, (heads + 2 kv_heads) d] holds
    the step's queries, keys and values, heads of one size d side by side; queries and keys take ``position``, keys and values go
    to their rows' cache slots (where the mixer owns the cache), and ``attn`` [T, heads d] receives softmax(scale q k) v over the
    keys each row may see. Which kernels run follows from the step's layout, the dtype and the sizes."""
    T = qkv.shape[0]
    exact = rt.exact
    mfma_heads = d % 16 == 0
    kv = ctx.kv(entry)
    plan = ctx.memo("gqa_attention.rows", lambda: RowPlan(ctx))
    table = position.table(ctx.n_positions)
    if table is None:
        hd = heads * d
        position.apply(ctx, qkv[:, :hd].unflatten(1, (heads, d)),
                            qkv[:, hd:hd + kv_heads * d].unflatten(1, (kv_heads, d)))
        table = ctx.identity_rotation(d)
    cos, sin = table
    common = (heads, kv_heads, d, window, scale)
    pow2_pages = kv.k.shape[2] >= ops.MIN_FAST_PAGE and kv.k.shape[2] & (kv.k.shape[2] - 1) == 0
    fast_prefill = d in ops.PREFILL_HEAD_DIMS
    # one new token per request: the decode kernel rotates it and writes its cache slot itself
    fused = (not exact and pow2_pages and mfma_heads and kv.owner and ctx.max_q_len == 1 and plan.long_runs is None
             and ops.can_fuse_rope_into_decode(d))
    if fused:
        pass
    elif kv.owner:
        ops.rope_kv_write(qkv, cos, sin, ctx.positions, heads, kv_heads, d, kv.slots, kv.k, kv.v)
    else:
        ops.rope_kv_write(qkv, cos, sin, ctx.positions, heads, kv_heads, d)
    if exact or not pow2_pages or not mfma_heads or (plan.long_runs is not None and not fast_prefill):
        # the exact path, and page or head sizes the bfloat16 kernels are not built for
        ops.paged_attention(attn, qkv, kv.k, kv.v, kv.block_table, ctx.req_of_token, ctx.positions, *common, exact)
    else:
        if plan.long_runs is not None:      # portions of prompts
            tiles, share, rows = plan.tiles(heads, kv_heads, d, window)
            ops.attention_prefill(attn, qkv, kv.k, kv.v, kv.block_table, tiles, *common, share=share, rows=rows)
        if plan.n_short:                    # single tokens and very short portions, all query heads of a key head together
            floats = ops.decode_scratch_floats(plan.n_short, heads, kv_heads, d, ctx.max_context, window)
            partial = ctx.scratch("attn_partial", (floats,), torch.float32) if floats else None
            # (one token per request and nothing else in the step: token i is request i)
            one_each = ctx.max_q_len == 1 and plan.short_rows is None and plan.long_runs is None
            ops.attention_decode(attn, qkv, kv.k, kv.v, kv.block_table, None if one_each else ctx.req_of_token, ctx.positions, *common,
                                 ctx.max_context, partial, rows=plan.short_rows, rope=(cos, sin, kv.slots) if fused else None)


NAMES = {"q": "q_proj.weight", "k": "k_proj.weight", "v": "v_proj.weight", "o": "o_proj.weight",
         "q_bias": "q_proj.bias", "k_bias": "k_proj.bias", "v_bias": "v_proj.bias", "o_bias": "o_proj.bias"}


def _padded_heads(t: torch.Tensor, heads: int, size: int, to: int, order=None) -> torch.Tensor:
    """Rows of ``t`` are ``heads`` heads of ``size`` channels: every head widened to ``to`` channels by zero rows, then
    its channels put in ``order`` (indices into the widened head)."""
    if size == to and order is None:
        return t
    rest = tuple(t.shape[1:])
    t = t.reshape(heads, size, *rest)
    if to > size:
        t = torch.cat([t, torch.zeros((heads, to - size, *rest), dtype=t.dtype, device=t.device)], dim=1)
    if order is not None:
        t = t[:, torch.tensor(order, dtype=torch.long, device=t.device)]
    return t.reshape(heads * to, *rest).contiguous()


class GQAAttention(Mixer):
    """params: prefix, hidden, heads, kv_heads, head_dim, qkv_bias, out_bias,
    window (None or a count of keys), position (PartSpec); optional: v_head_dim (the size of a value head, default
    head_dim), scale (what scores are multiplied by, default 1/sqrt(head_dim)), names (tensor names after the prefix
    for q, k, v, o and their biases, default the *_proj ones), init (the rule random weights are drawn by).

    The kernels know one head size d. Where query/key and value heads differ in size, or the size is none the
    prefill kernel is built for, every head is widened to a common d with zero rows in its projection (zero columns
    in the output matrix): products with zeros change nothing."""
    capturable = True   # native kernels on the current stream only: a decode step may be graph-captured

    @classmethod
    def tensors(cls, spec):
        p = spec.params
        names, init = {**NAMES, **p.get("names", {})}, p.get("init", "matrix")
        dv = p.get("v_head_dim") or p["head_dim"]
        pre, h, qd, kd, vd, od = p["prefix"], p["hidden"], p["heads"] * p["head_dim"], p["kv_heads"] * p["head_dim"], p["kv_heads"] * dv, p["heads"] * dv
        out = {pre + names["q"]: TensorRule((qd, h), init), pre + names["k"]: TensorRule((kd, h), init),
               pre + names["v"]: TensorRule((vd, h), init), pre + names["o"]: TensorRule((h, od), init)}
        if p.get("qkv_bias", False):
            out.update({pre + names["q_bias"]: TensorRule((qd,), "bias"), pre + names["k_bias"]: TensorRule((kd,), "bias"),
                        pre + names["v_bias"]: TensorRule((vd,), "bias")})
        if p.get("out_bias", False):
            out[pre + names["o_bias"]] = TensorRule((h,), "bias")
        return out

    @staticmethod
    def common_head_size(qk: int, v: int) -> int:
        """The one head size the kernels run with: the larger of the two; when they differ, or the size is odd, the
        next size the prefill kernel is built for, if there is one."""
        d = max(qk, v)
        d += d % 2
        if qk != v or d != qk:
            d = next((n for n in ops.PREFILL_HEAD_DIMS if n >= d), d)
        return d

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        p = spec.params
        self.hidden, self.heads, self.kv_heads = int(p["hidden"]), int(p["heads"]), int(p["kv_heads"])
        self.qk_dim = int(p["head_dim"])
        self.v_dim = int(p.get("v_head_dim") or self.qk_dim)
        self.d = self.common_head_size(self.qk_dim, self.v_dim)
        self.window = p.get("window")
        if self.kv_heads <= 0 or self.heads % self.kv_heads:
            raise AlofaError("unsupported", "kv_heads must be positive and divide heads", f"heads={self.heads} kv_heads={self.kv_heads}")
        if self.d % 2 or not 2 <= self.d <= ops.MAX_HEAD_DIM:
            raise AlofaError("unsupported", f"the attention kernels take even head sizes up to {ops.MAX_HEAD_DIM}", f"head_dim={self.d}")
        # (the matrix-core kernels take head sizes in steps of 16; any other even size runs on the always-valid kernels, in both dtypes)
        self.mfma_heads = self.d % 16 == 0
        if self.window is not None and self.window <= 0:
            raise AlofaError("invalid_argument", "an attention window must be positive", f"window={self.window}")
        pre, names = p["prefix"], {**NAMES, **p.get("names", {})}
        position = p["position"]
        if self.d != self.qk_dim:
            position = part_class("position", position.kind).for_head(position, self.d)
        self.position = build_part("position", position, weights, rt)
        order = self.position.channel_order()      # (the order of a head's channels in which the encoding's pairs lie as the kernels pair them)
        sizes = {"q": (self.heads, self.qk_dim, order), "k": (self.kv_heads, self.qk_dim, order), "v": (self.kv_heads, self.v_dim, None)}
        mats = [_padded_heads(weights[pre + names[n]], *sizes[n][:2], self.d, sizes[n][2]) for n in ("q", "k", "v")]
        if len({m.dtype for m in mats}) > 1:
            mats = [m.float() for m in mats]
        self.w_qkv = rt.matrix(torch.cat(mats, dim=0))
        self.b_qkv = (rt.vector(torch.cat([_padded_heads(weights[pre + names[n + "_bias"]].float(), *sizes[n][:2], self.d, sizes[n][2]) for n in ("q", "k", "v")]))
                      if p.get("qkv_bias", False) else None)
        w_o = weights[pre + names["o"]]
        if self.d != self.v_dim:      # zero columns where the value heads were widened
            w_o = _padded_heads(w_o.t(), self.heads, self.v_dim, self.d).t()
        self.w_o = rt.matrix(w_o)
        self.b_o = rt.vector(weights[pre + names["o_bias"]]) if p.get("out_bias", False) else None
        # float32 1 / sqrt(float32 d), as the reference forms it (scalar.mojo:421), unless the configuration gives the factor
        self.scale = float(p["scale"]) if p.get("scale") is not None else float(np.float32(1.0) / np.sqrt(np.float32(self.qk_dim)))
        self.qkv_width = (self.heads + 2 * self.kv_heads) * self.d
        # an encoding applied by other code (``apply``) is captured only if it says that it may be: native kernels or
        # library calls on the current stream that allocate nothing and record no memset
        self.capturable = self.position.table(1) is not None or bool(getattr(self.position, "capturable", False))

    def cache_need(self):
        return CacheNeed.keys_and_values(self.kv_heads, self.d, self.window)

    def prepare(self, n_positions):
        self.position.table(n_positions)       # built up to the context bound once, so that it never moves afterwards

    def fuses_norm(self, norm, rows):
        return (not self.rt.exact and norm.as_rmsnorm() is not None
                and ops.can_fuse_norm(rows, self.w_qkv, self.rt.dtype))

    @property
    def gives_normed(self):
        return self.b_o is None

    def forward(self, ctx, entry, x, residual, norm=None, then=None, out=None):
        """``out`` (float32, the residual's shape): the mix is stored there instead of being added to the residual."""
        T = residual.shape[0]
        exact = self.rt.exact
        qkv = ctx.scratch("qkv", (T, self.qkv_width), self.rt.dtype)
        if norm is not None:      # the input norm rides on the product
            ops.gemm(qkv, residual, self.w_qkv, self.b_qkv, norm=norm.as_rmsnorm())
        else:
            ops.gemm(qkv, x, self.w_qkv, self.b_qkv, exact=exact)
        attn = ctx.scratch("attn", (T, self.heads * self.d), self.rt.dtype)
        paged_attend(ctx, entry, qkv, attn, self.heads, self.kv_heads, self.d, self.window, self.scale, self.position, self.rt)
        if out is not None:
            ops.gemm(out, attn, self.w_o, self.b_o, exact=exact)
        elif self.b_o is not None:
            proj = ctx.scratch("attn_proj", (T, self.hidden), torch.float32)
            ops.gemm(proj, attn, self.w_o, self.b_o, exact=exact)
            residual.add_(proj)
        else:      # (then: the norm behind this part, left in the rows given with it)
            ops.gemm(residual, attn, self.w_o, add_to_out=True, exact=exact, then_norm=_then(then))


def _then(then):
    """(norm, rows) as ``ops.gemm(then_norm=)`` wants it, for norms that are plain RMSNorms; any other norm runs here
    by itself afterwards, which ``ops.gemm`` cannot do for it: such parts are not asked (``gives_normed`` holds only
    for RMSNorm in the blocks of this package)."""
    if then is None:
        return None
    norm, rows = then
    weight, eps = norm.as_rmsnorm()
    return weight, eps, rows


register_part("mixer", "gqa_attention", GQAAttention)

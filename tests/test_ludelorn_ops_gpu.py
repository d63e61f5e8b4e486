"""The kernels behind Ludelorn's parts, each alone against the plain functions (float64 on the host): norms and turns of queries and keys
on their way into the pages, pooled blocks, attention over a window with blocks, bias, sink and gates (the always-valid kernel against the
plain softmax, the matrix-core kernel against both), the short convolution with its state over portions, the state-space operands and
read-out, the sum of normed branches, the activation."""
import math

import numpy as np
import pytest
import torch

from plain import ludelorn as pl

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
F = torch.float64


def tol(dtype):
    return 2e-5 if dtype is torch.float32 else 2e-2


def close(got, want, dtype, what):
    got, want = got.detach().double().cpu(), want.double().cpu()
    err = (got - want).abs().max().item()
    assert err <= tol(dtype) * max(1.0, want.abs().max().item()), f"{what}: {err}"


class Pages:
    """Keys and values of a few requests scattered over pages in a shuffled order, with the tables the kernels read."""

    def __init__(self, lengths, G, d, dv, S, dtype, seed, pool=None):
        g = torch.Generator().manual_seed(seed)
        self.lengths, self.S, self.G, self.d, self.dv, self.pool = lengths, S, G, d, dv, pool
        n_pages = sum((n + S - 1) // S for n in lengths) + 3
        order = torch.randperm(n_pages, generator=g).tolist()
        width = max((n + S - 1) // S for n in lengths)
        self.table = torch.full((len(lengths), width), -1, dtype=torch.int32)
        self.k = [torch.randn(n, G, d, generator=g).to(dtype) for n in lengths]
        self.v = [torch.randn(n, G, dv, generator=g).to(dtype) for n in lengths]
        self.kc = torch.zeros(n_pages, G, S, d, dtype=dtype)
        self.vc = torch.zeros(n_pages, G, dv, S, dtype=dtype)
        for r, n in enumerate(lengths):
            for b in range((n + S - 1) // S):
                page = order.pop()
                self.table[r, b] = page
                rows = slice(b * S, min(n, (b + 1) * S))
                m = rows.stop - rows.start
                self.kc[page, :, :m] = self.k[r][rows].transpose(0, 1)
                self.vc[page, :, :, :m] = self.v[r][rows].permute(1, 2, 0)
        self.places = (S - 1) // pool + 1 if pool else 0
        if pool:
            self.pk = torch.zeros(n_pages, G, self.places, d, dtype=dtype)
            self.pv = torch.zeros(n_pages, G, dv, self.places, dtype=dtype)

    def cuda(self):
        for n in ("table", "kc", "vc", "pk", "pv"):
            if hasattr(self, n):
                setattr(self, n, getattr(self, n).to(DEV))
        return self


def plain_span(q, k, v, p, window, scale, pool=None, bias=None, sink=None, store=lambda x: x):
    """One query row [H, d] at position p over its request's keys [n, G, d] and values: float64."""
    H, G = q.shape[0], k.shape[1]
    per = H // G
    lo = max(0, p - window + 1) if window else 0
    keys, vals = [k[lo:p + 1].double()], [v[lo:p + 1].double()]
    dist = [p - j for j in range(lo, p + 1)]
    if pool:
        nb = max(0, (p - window + 1) // pool) if p - window + 1 >= pool else 0
        if nb:
            keys.append(store(k[:nb * pool].double().view(nb, pool, G, -1).mean(1)))
            vals.append(store(v[:nb * pool].double().view(nb, pool, G, -1).mean(1)))
            dist += [None] * nb
    keys, vals = torch.cat(keys), torch.cat(vals)
    out = torch.zeros(H, v.shape[2], dtype=F)
    for h in range(H):
        s = keys[:, h // per] @ q[h].double() * scale
        if bias is not None:
            s = s + torch.tensor([0.0 if x is None else float(bias[h, min(x, bias.shape[1] - 1)]) for x in dist], dtype=F)
        top = s.max() if sink is None else max(s.max(), sink[h].double())
        e = torch.exp(s - top)
        total = e.sum() + (torch.exp(sink[h].double() - top) if sink is not None else 0.0)
        out[h] = (e / total) @ vals[:, h // per]
    return out


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("scope,weights,turned,values_are_keys", [("head", True, True, False), ("all", True, True, False), ("head", False, False, True), (None, False, True, False)])
def test_norm_turn_write(dtype, scope, weights, turned, values_are_keys):
    from alofa_amd import ops
    torch.manual_seed(1)
    T, H, G, d, true_d, S = 37, 3, 2, 16, 12, 8
    dv = d
    eps = 1e-5
    width = H * d + G * d + (0 if values_are_keys else G * dv)
    x = torch.randn(T, width).to(dtype)
    xv = x.view(T, -1)
    # (heads widened from 12 to 16 channels with zeros, as the mixer's projection leaves them)
    for u in range(H + G):
        xv[:, u * d + true_d:(u + 1) * d] = 0
    pos = torch.randint(0, 50, (T,), dtype=torch.int32)
    half = d // 2
    ang = torch.rand(64, half, dtype=F) * 6
    cos, sin = torch.cos(ang).float(), torch.sin(ang).float()
    wq = torch.rand(d if scope == "head" else H * d) + 0.5 if weights else None
    wk = torch.rand(d if scope == "head" else G * d) + 0.5 if weights else None
    slots = torch.randperm(6 * S)[:T].to(torch.int64)
    kc, vc = torch.zeros(6, G, S, d, dtype=dtype, device=DEV), torch.zeros(6, G, dv, S, dtype=dtype, device=DEV)
    xd = x.clone().to(DEV)
    code = {None: ops.NORM_NONE, "head": ops.NORM_HEAD, "all": ops.NORM_ALL}[scope]
    factors = torch.zeros(T, 2, dtype=torch.float64, device=DEV)
    ops.norm_turn_write(xd, pos.to(DEV), (cos.to(DEV), sin.to(DEV)) if turned else None, H, G, d, dv, code, wq.to(DEV) if weights else None, wk.to(DEV) if weights else None,
                        eps, dtype is torch.float32, slots.to(DEV), kc, vc, values_are_keys, factors, true_d=true_d)
    xs = x.double()
    q, k = xs[:, :H * d].view(T, H, d), xs[:, H * d:(H + G) * d].view(T, G, d)

    def normed(t, w, n_heads):
        if scope == "head":
            t = t / torch.sqrt((t * t).sum(-1, keepdim=True) / true_d + eps)
            return t * w.double() if w is not None else t
        if scope == "all":
            flat = t.reshape(T, -1)
            flat = flat / torch.sqrt((flat * flat).sum(-1, keepdim=True) / (n_heads * true_d) + eps) * w.double()
            return flat.view(T, n_heads, d)
        return t

    def turn(t):
        if not turned:
            return t
        c, s = cos.double()[pos.long()][:, None, :], sin.double()[pos.long()][:, None, :]
        u, v = t[..., :half], t[..., half:]
        return torch.cat([u * c - v * s, v * c + u * s], dim=-1)
    want_q, want_k = turn(normed(q, wq, H)), turn(normed(k, wk, G))
    close(xd[:, :H * d].view(T, H, d), want_q, dtype, "queries")
    got_k = kc.view(-1, G, S, d).permute(0, 2, 1, 3).reshape(-1, G, d)[slots.to(DEV)]
    close(got_k, want_k, dtype, "keys in their pages")
    want_v = k if values_are_keys else xs[:, (H + G) * d:].view(T, G, dv)
    got_v = vc.permute(0, 3, 1, 2).reshape(-1, G, dv)[slots.to(DEV)]
    close(got_v, want_v, dtype, "values in their pages")


CASES = [
    # lengths, H, G, d, window, pool, bias rows/far, sink, gate
    dict(lengths=(70, 23, 130), H=4, G=2, d=32, window=24, pool=5, S=16),
    dict(lengths=(90, 40), H=4, G=4, d=16, window=33, pool=16, S=16, gate="channel"),
    dict(lengths=(150,), H=6, G=2, d=48, window=20, pool=7, S=8, gate="head"),
    dict(lengths=(60, 61), H=8, G=2, d=16, window=18, bias=(8, 14.0), sink=True, S=16, gate="head"),
    dict(lengths=(45, 100), H=2, G=1, d=64, window=31, bias=(16, 20.0), sink=True, S=32),
    dict(lengths=(80,), H=3, G=3, d=80, window=1, sink=True, S=16),
    dict(lengths=(50, 77), H=2, G=2, d=16, window=9, pool=1, S=16, gate="channel"),
]


@pytest.mark.parametrize("case", CASES, ids=[str(i) for i in range(len(CASES))])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_over_a_window_with_blocks_bias_and_sink(case, dtype):
    """Every row of every request as a query at its own position: the always-valid kernel against the plain softmax; in bfloat16 the matrix-core
    kernel against both, with the rows as runs of up to sixteen and as single rows; the pooled blocks as ``pool_blocks`` leaves them."""
    from alofa_amd import ops
    from alofa_amd.parts.window import distance_buckets
    H, G, d, window, S = case["H"], case["G"], case["d"], case["window"], case["S"]
    pool = case.get("pool")
    pages = Pages(case["lengths"], G, d, d, S, dtype, seed=5, pool=pool).cuda()
    g = torch.Generator().manual_seed(9)
    rows = [(r, p) for r, n in enumerate(case["lengths"]) for p in range(n)]
    T = len(rows)
    q = (torch.randn(T, H * d, generator=g) * 0.7).to(dtype)
    positions = torch.tensor([p for _, p in rows], dtype=torch.int32, device=DEV)
    req = torch.tensor([r for r, _ in rows], dtype=torch.int32, device=DEV)
    scale = 2.0 / math.sqrt(d)
    bias = sink = gate = None
    if case.get("bias"):
        n_rows, far = case["bias"]
        table = torch.randn(n_rows, H, generator=g) * 2
        bias = table[torch.tensor(distance_buckets(n_rows, far, min(window, int(math.ceil(far)) + 1)))].t().contiguous()
    if case.get("sink"):
        sink = torch.randn(H, generator=g) * 3
    kind = {None: ops.GATE_NONE, "channel": ops.GATE_CHANNEL, "head": ops.GATE_HEAD}[case.get("gate")]
    if kind:
        gate = torch.randn(T, H * d if kind == ops.GATE_CHANNEL else H, generator=g).to(dtype)
    exact = dtype is torch.float32
    pooled = None
    if pool:
        ops.pool_blocks(pages.kc, pages.vc, pages.pk, pages.pv, pages.table, pages.table, req, positions, G, d, d, pool, exact)
        pooled = (pages.pk, pages.pv, pages.table, pool)
    dev = lambda t: None if t is None else t.to(DEV)
    out = torch.zeros(T, H * d, dtype=dtype, device=DEV)
    ops.span_attention(out, q.to(DEV), pages.kc, pages.vc, pages.table, req, positions, H, G, d, d, window, scale, exact, pooled=pooled, bias=dev(bias), sink=dev(sink),
                       gate=dev(gate), gate_kind=kind)
    store = (lambda x: x) if exact else pl.to_bfloat16
    want = torch.stack([plain_span(q[t].view(H, d), pages.k[r], pages.v[r], p, window, scale, pool, bias, sink, store) for t, (r, p) in enumerate(rows)]).reshape(T, H * d)
    if kind == ops.GATE_CHANNEL:
        want = want * torch.sigmoid(gate.double())
    elif kind == ops.GATE_HEAD:
        want = (want.view(T, H, d) * torch.sigmoid(gate.double())[:, :, None]).reshape(T, H * d)
    close(out, want, dtype, "always-valid kernel")
    if exact or d % 16:
        return
    runs, row = [], 0
    for r, n in enumerate(case["lengths"]):
        for q0 in range(0, n, 16):
            runs.append((r, row + q0, min(16, n - q0)))
        row += n
    # (runs that start anywhere: the first run of every request cut in two unequal ones)
    ragged = []
    for r, row0, n in runs:
        ragged += [(r, row0, 5), (r, row0 + 5, n - 5)] if n > 5 else [(r, row0, n)]
    for what, tiles in (("runs of sixteen", runs), ("ragged runs", ragged), ("single rows", None)):
        fast = torch.zeros(T, H * d, dtype=dtype, device=DEV)
        ops.span_attention_mfma(fast, q.to(DEV), pages.kc, pages.vc, pages.table, None if tiles is None else torch.tensor(tiles, dtype=torch.int32, device=DEV), req, positions,
                                H, G, d, window, scale, pooled=pooled, bias=dev(bias), sink=dev(sink), gate=dev(gate), gate_kind=kind)
        close(fast, want, dtype, f"matrix-core kernel, {what}")
        assert (fast.float() - out.float()).abs().max().item() <= 2e-2 * max(1.0, want.abs().max().item())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("taps", [1, 2, 4])
def test_the_convolution_and_its_state_over_portions(dtype, taps):
    """Two requests in portions of unequal size, a slot's state carried from step to step; a step of single rows through the fused kernel."""
    from alofa_amd import ops
    torch.manual_seed(3)
    H, G, N, dv = 3, 1, 5, 4
    C = H * dv + 2 * G * N
    lengths = (23, 9)
    x = [torch.randn(n, C + 3).to(dtype) for n in lengths]      # (rows with a stride: three more columns)
    w, b = torch.randn(C, taps) * 0.5, torch.randn(C)
    want = [pl.silu(pl.causal_conv(t[:, :C].double(), w.double(), b.double())) for t in x]
    state = torch.zeros(4, taps - 1, C, dtype=dtype, device=DEV)
    slots = torch.tensor([2, 0], dtype=torch.int32, device=DEV)
    exact = dtype is torch.float32
    at, got = [0, 0], [[], []]
    for step in ((5, 2), (1, 1), (9, 3), (1, 1), (7, 2)):
        rows_in = torch.cat([x[r][at[r]:at[r] + n] for r, n in enumerate(step)]).to(DEV)
        T = sum(step)
        single = all(n == 1 for n in step)
        rows = ops.RowsOfRequests(slots, None if single else torch.tensor([0, step[0], T], dtype=torch.int32, device=DEV),
                                  None if single else torch.tensor([0] * step[0] + [1] * step[1], dtype=torch.int32, device=DEV), 2, T, 4)
        out = torch.zeros(T, C, dtype=dtype, device=DEV)
        if single:
            dt = torch.randn(T, H).to(dtype).to(DEV)
            ops_out = [torch.zeros(T, H * N, device=DEV) for _ in range(2)] + [torch.zeros(T, H * dv, device=DEV), torch.zeros(T, H * N, device=DEV)]
            dt_bias, a_log = torch.randn(H, device=DEV), torch.randn(H, device=DEV)
            ops.ssd_step(out, rows_in[:, :C], w.to(DEV), b.to(DEV), state if taps > 1 else None, rows, *ops_out, dt, dt_bias, a_log, H, G, N, dv, exact)
            apart = [torch.zeros_like(t) for t in ops_out]
            ops.ssd_operands(*apart, out, dt, dt_bias, a_log, H, G, N, dv, exact)
            for a_, b_ in zip(ops_out, apart):
                assert torch.equal(a_, b_)
        else:
            none = torch.zeros(4, 0, C, dtype=dtype, device=DEV)
            ops.conv_bias_act(out, rows_in[:, :C], w.to(DEV), b.to(DEV), state if taps > 1 else none, rows, silu=True, exact=exact)
            if taps > 1:
                ops.conv_keep(state, rows_in[:, :C], rows)
        o = 0
        for r, n in enumerate(step):
            got[r].append(out[o:o + n].cpu())
            o += n
            at[r] += n
    for r in range(2):
        close(torch.cat(got[r]), want[r][:at[r]], dtype, f"request {r}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_state_space_operands_and_read_out(dtype):
    from alofa_amd import ops
    torch.manual_seed(4)
    T, H, G, N, dv, parts = 11, 6, 2, 5, 4, 3
    inner = H * dv
    xbc = torch.randn(T, inner + 2 * G * N).to(dtype)
    dt, dt_bias, a_log = (torch.randn(T, H) * 3).to(dtype), torch.randn(H), torch.randn(H)
    qf, kf, decay, vf = torch.zeros(T, H * N, device=DEV), torch.zeros(T, H * N, device=DEV), torch.zeros(T, H * N, device=DEV), torch.zeros(T, inner, device=DEV)
    exact = dtype is torch.float32
    ops.ssd_operands(qf, kf, vf, decay, xbc.to(DEV), dt.to(DEV), dt_bias.to(DEV), a_log.to(DEV), H, G, N, dv, exact)
    step = pl.softplus(dt.double() + dt_bias.double())
    B = xbc[:, inner:inner + G * N].double().view(T, G, N).repeat_interleave(H // G, 1)
    Cq = xbc[:, inner + G * N:].double().view(T, G, N).repeat_interleave(H // G, 1)
    close(kf.view(T, H, N), step[:, :, None] * B, torch.float32, "keys")
    close(qf.view(T, H, N), Cq, torch.float32, "queries")
    close(decay.view(T, H, N), torch.exp(-torch.exp(a_log.double()) * step)[:, :, None].expand(T, H, N), torch.float32, "decays")
    close(vf, xbc[:, :inner].double(), torch.float32, "values")
    o = torch.randn(2, T, inner)
    z, skip, weight = torch.randn(T, inner).to(dtype), torch.randn(H), torch.rand(inner) + 0.5
    out = torch.zeros(T, inner, dtype=dtype, device=DEV)
    ops.ssd_finish(out, o.to(DEV), xbc[:, :inner].to(DEV), z.to(DEV), skip.to(DEV), weight.to(DEV), H, dv, parts, 1e-5, exact, parts=2)
    y = (o.double().sum(0) + skip.double().repeat_interleave(dv) * xbc[:, :inner].double()) * pl.silu(z.double())
    y = pl.rms(y.view(T, parts, inner // parts), 1e-5).reshape(T, inner) * weight.double()
    close(out, y, dtype, "read-out")


@pytest.mark.parametrize("exact", [True, False])
def test_the_sum_of_normed_branches(exact):
    from alofa_amd import ops
    torch.manual_seed(6)
    T, h = 7, 300
    a, b, wa, wb, scale, nw = torch.randn(T, h) * 3, torch.randn(T, h), torch.rand(h) + 0.5, torch.rand(h) + 0.5, torch.randn(h), torch.rand(h) + 0.5
    res = torch.randn(T, h)
    want = 0.5 * (pl.rms(a.double(), 1e-5) * wa.double() + pl.rms(b.double(), 1e-5) * wb.double())
    out = torch.zeros(T, h, device=DEV)
    ops.rms_pair_sum(out, a.to(DEV), wa.to(DEV), 0.5, b.to(DEV), wb.to(DEV), 0.5, 1e-5, exact)
    close(out, want, torch.float32, "sum apart")
    stream = res.clone().to(DEV)
    normed = torch.zeros(T, h, dtype=torch.float32 if exact else torch.bfloat16, device=DEV)
    ops.rms_pair_add_norm(stream, a.to(DEV), wa.to(DEV), 0.5, b.to(DEV), wb.to(DEV), 0.5, scale.to(DEV), 1e-5, exact, then_norm=(nw.to(DEV), 1e-6, normed))
    new = res.double() + scale.double() * want
    close(stream, new, torch.float32, "sum into the stream")
    close(normed, pl.rms(new, 1e-6) * nw.double(), normed.dtype, "the norm behind it")
    alone = res.clone().to(DEV)
    ops.rms_pair_add_norm(alone, a.to(DEV), wa.to(DEV), 0.5, b.to(DEV), wb.to(DEV), 0.5, None, 1e-5, exact)
    close(alone, res.double() + want, torch.float32, "sum without factors")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gelu(dtype):
    from alofa_amd import ops
    x = (torch.linspace(-9, 9, 1001).view(7, 143)).to(dtype)
    out = torch.zeros_like(x, device=DEV)
    ops.activation(out, x.to(DEV), ops.GELU_TANH, exact=dtype is torch.float32)
    close(out, pl.gelu_tanh(x.double()), dtype, "gelu")

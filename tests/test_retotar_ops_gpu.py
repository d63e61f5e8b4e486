"""Each kernel of the Retotar mechanisms alone against the plain function of the same equation: rows of several requests in one
call, pages in a shuffled order, state carried from call to call, sizes that no tile divides."""
import numpy as np
import pytest
import torch

from plain import retotar as pt
from test_recurrent_ops_gpu import DEV, cuts, dev, rows_of

pytestmark = pytest.mark.gpu

F = torch.float64


def tables(base, n, positions, factor=1.0):
    """(cos, sin) float32 [positions, n / 2] as the engine's rotary part makes them."""
    from alofa_amd.config.base import PartSpec
    from alofa_amd.parts.base import Runtime, build_part
    rt = Runtime(torch.device(DEV), torch.float32)
    return build_part("position", PartSpec("rotary", {"theta": base, "head_dim": n, "factor": factor}), {}, rt).table(positions)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,d,dv,dims,window", [(4, 2, 16, 24, 8, 20), (3, 1, 24, 40, 24, 7), (2, 2, 32, 16, 2, None), (8, 4, 64, 32, 32, 33),
                                                  (5, 5, 10, 6, 4, 16), (12, 3, 128, 128, 64, 48), (6, 6, 9, 2, 6, 1), (4, 2, 32, 32, 16, 20),
                                                  (6, 6, 16, 16, 8, None), (8, 2, 64, 64, 32, 33), (16, 1, 48, 48, 48, 5), (4, 2, 96, 96, 32, 40),
                                                  (2, 1, 256, 256, 64, 30), (34, 2, 16, 16, 8, 25), (4, 2, 80, 80, 16, 30), (32, 4, 256, 256, 64, 30)])
def test_attention_over_shuffled_pages_in_portions(H, G, d, dv, dims, window, dtype):
    """Three requests of unequal length whose rows come in portions, mixed in every call; queries and keys turned and normed, values
    turned and the result turned back, the heads' weights mixed, the gate: against the plain functions on the whole sequences. Where
    the matrix-core kernels take the sizes (bfloat16, heads of one size in steps of 16), the same rows also go through them, once per
    value head, and through the kernel that mixes afterwards."""
    from alofa_amd import ops
    g = torch.Generator().manual_seed(H * 100 + d)
    exact = dtype is torch.float32
    lengths, page, base, factor, scale, eps = [70, 33, 51], 16, 1000.0, 3.0, 0.3, 1e-5
    store = pt._id if exact else pt.to_bfloat16
    n_pages = sum((n + page - 1) // page for n in lengths)
    order = torch.randperm(n_pages, generator=g).tolist()
    table = torch.full((3, 8), -1, dtype=torch.int32)
    for r, n in enumerate(lengths):
        for b in range((n + page - 1) // page):
            table[r, b] = order.pop()
    kc = torch.zeros(n_pages, G, page, d, dtype=dtype, device=DEV)
    vc = torch.zeros(n_pages, G, dv, page, dtype=dtype, device=DEV)
    talk = torch.eye(H, dtype=F) + 0.3 * torch.randn(H, H, generator=g, dtype=F)
    qk_t, v_t = tables(base, dims, 128, factor), tables(base, dv, 128)
    width = H * d + G * (d + dv)
    raw = [store(torch.randn(n, width + H * dv, generator=g, dtype=F)) for n in lengths]      # per request: q, k, v heads and the gate's rows
    # the plain result, request by request
    want = []
    for x in raw:
        n = x.shape[0]
        pos = torch.arange(n)
        q = store(pt.unit_rms(pt.turn_halves(x[:, :H * d].view(n, H, d), pos, dims, base, factor), eps))
        k = store(pt.unit_rms(pt.turn_halves(x[:, H * d:(H + G) * d].view(n, G, d), pos, dims, base, factor), eps))
        v = store(pt.turn_halves(x[:, (H + G) * d:width].view(n, G, dv), pos, dv, base))
        s = torch.einsum("ihc,jhc->hij", q, k.repeat_interleave(H // G, dim=1)) * scale
        seen = pos[None, :] <= pos[:, None]
        if window is not None:
            seen = seen & (pos[:, None] - pos[None, :] < window)
        p = torch.einsum("hg,gij->hij", talk, torch.softmax(s.masked_fill(~seen[None], float("-inf")), -1))
        o = pt.turn_halves(torch.einsum("hij,jhc->ihc", p, v.repeat_interleave(H // G, dim=1)), pos, dv, base, sign=-1.0)
        want.append(o.reshape(n, H * dv) * torch.sigmoid(x[:, width:]))
    # the kernels, in calls that mix portions of the three requests
    got = [torch.zeros(n, H * dv, dtype=F) for n in lengths]
    fast = not exact and d == dv and d in ops.PREFILL_HEAD_DIMS
    got_fast = [torch.zeros(n, H * dv, dtype=F) for n in lengths]
    done = [0, 0, 0]
    plans = [cuts(70, (31, 2, 1, 17)), cuts(33, (2, 9, 1, 1)), cuts(51, (16, 1, 20, 3))]
    for step in range(max(len(p) for p in plans)):
        live = [(r, *plans[r][step]) for r in range(3) if step < len(plans[r])]
        rows = torch.cat([raw[r][a:b] for r, a, b in live]).to(dtype).to(DEV).contiguous()
        positions = torch.tensor([p for r, a, b in live for p in range(a, b)], dtype=torch.int32, device=DEV)
        req = torch.tensor([r for r, a, b in live for _ in range(a, b)], dtype=torch.int32, device=DEV)
        slots = torch.tensor([int(table[r, p // page]) * page + p % page for r, a, b in live for p in range(a, b)], dtype=torch.int64, device=DEV)
        ops.turn_norm_write(rows[:, :width], positions, qk_t, v_t, H, G, d, dv, eps, True, exact, slots, kc, vc)
        out = torch.empty(rows.shape[0], H * dv, dtype=dtype, device=DEV)
        ops.talking_attention(out, rows[:, :H * d], kc, vc, table.to(DEV), req, positions, H, G, d, dv, window, scale, dev(talk.numpy()), v_t, rows[:, width:], exact)
        if fast:
            # portions of more than a few rows through the prefill kernel in runs of up to 64, the others row by row through the decode kernel
            runs, short, row = [], [], 0
            for r, a, b in live:
                if b - a > ops.DECODE_MAX_Q:
                    runs += [(r, row + q0, min(64, b - a - q0), a + q0) for q0 in range(0, b - a, 64)]
                else:
                    short += list(range(row, row + b - a))
                row += b - a
            applied = torch.full((G, rows.shape[0], H * dv), float("nan"), device=DEV)
            for c in range(G):
                if runs:
                    tiles = torch.tensor(ops.pair_tiles(runs, window, H), dtype=torch.int32, device=DEV)
                    ops.attention_prefill(applied[c], rows[:, :H * d], kc, vc, table.to(DEV), tiles, H, G, d, window, scale, v_head=c, fine_weights=True)
                if short:
                    floats = ops.decode_scratch_floats(len(short), H, G, d, 128, window)
                    ops.attention_decode(applied[c], rows[:, :H * d], kc, vc, table.to(DEV), req, positions, H, G, d, window, scale, 128,
                                         torch.empty(max(floats, 1), device=DEV), rows=torch.tensor(short, dtype=torch.int32, device=DEV), v_head=c, fine_weights=True)
            # ... and all value heads in one launch of each kernel: the same numbers (the keys may be cut into other parts)
            together = torch.full((G, rows.shape[0], H * dv), float("nan"), device=DEV)
            if runs:
                ops.attention_prefill(together, rows[:, :H * d], kc, vc, table.to(DEV), tiles, H, G, d, window, scale, fine_weights=True, all_value_heads=True)
            if short:
                floats = ops.decode_scratch_floats(len(short) * G, H, G, d, 128, window)
                ops.attention_decode(together, rows[:, :H * d], kc, vc, table.to(DEV), req, positions, H, G, d, window, scale, 128,
                                     torch.empty(max(floats, 1), device=DEV), rows=torch.tensor(short, dtype=torch.int32, device=DEV), fine_weights=True, all_value_heads=True)
            assert (together - applied).abs().max().item() <= 1e-5 * max(1.0, applied.abs().max().item())
            out_fast = torch.empty_like(out)
            ops.talk_mix(out_fast, applied, positions, H, G, dv, dev(talk.numpy()), v_t, rows[:, width:])
        at = 0
        for r, a, b in live:
            got[r][a:b] = out[at:at + b - a].double().cpu()
            if fast:
                got_fast[r][a:b] = out_fast[at:at + b - a].double().cpu()
            at += b - a
            done[r] = b
    assert done == lengths
    for r in range(3):
        for which, rows_got in (("a block per row", got), ("matrix cores", got_fast)) if fast else (("a block per row", got),):
            err = (rows_got[r] - want[r]).abs().max().item()
            assert err <= (2e-5 if exact else 3e-2) * max(1.0, want[r].abs().max().item()), f"request {r} ({which}): {err}"


@pytest.mark.parametrize("exact", [True, False])
@pytest.mark.parametrize("E,passing,groups,keep,top", [(18, 2, 2, 1, 3), (8, 3, 4, 2, 3), (3, 0, 1, 1, 1), (4, 1, 2, 1, 2), (100, 20, 10, 3, 7), (512, 0, 8, 8, 5), (9, 2, 3, 2, 6)])
def test_the_choice_among_experts_in_groups(E, passing, groups, keep, top, exact):
    from alofa_amd import ops
    g = torch.Generator().manual_seed(E)
    T = 37
    z = torch.randn(T, E, generator=g, dtype=torch.float32) * 2.0
    corr = torch.randn(E, generator=g, dtype=torch.float32) * (0.5 / E)
    chosen, weights = pt.choose_experts(z.double(), corr.double(), {"top": top, "groups": {"count": groups, "keep": keep}})
    dense, ch, wt, pw = (torch.empty(T, E - passing, device=DEV), torch.empty(T, top, dtype=torch.int32, device=DEV), torch.empty(T, top, device=DEV),
                         torch.empty(T, device=DEV))
    ops.route_groups(z.to(DEV), corr.to(DEV), dense, ch, wt, pw, top, passing, groups, keep, exact=exact)
    assert torch.equal(ch.cpu().long(), chosen)
    assert (wt.cpu().double() - weights).abs().max() <= 1e-6
    full = torch.zeros(T, E, dtype=F).scatter_(1, chosen, weights)
    assert (dense.cpu().double() - full[:, :E - passing]).abs().max() <= 1e-6
    assert (pw.cpu().double() - full[:, E - passing:].sum(1)).abs().max() <= 1e-6


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,d,dv", [(2, 24, 16), (4, 64, 128), (5, 5, 3), (1, 32, 32), (3, 16, 63)])
def test_the_memory_with_gates_in_portions_of_two_requests(H, d, dv, dtype):
    """Gates with their running maximum, the recurrence with the normaliser as one more value channel, the division, the head norm and
    the gate, against the plain memory; two requests in unequal portions (single rows among them) within the same calls."""
    from alofa_amd import ops
    g = torch.Generator().manual_seed(d + dv)
    exact, cap, eps = dtype is torch.float32, 7.0, 1e-5
    store = pt._id if exact else pt.to_bfloat16
    width = 2 * H * d + 2 * H * dv
    lengths = [290, 41]      # (portions of one row, of fewer and of more than a wavefront's 64 rows, and of exactly 128)
    raw = [store(torch.randn(n, width, generator=g, dtype=F)) for n in lengths]
    zs = [torch.randn(n, 2 * H, generator=g, dtype=torch.float32) * 3.0 for n in lengths]
    zs[0][:, H:] += 4.0      # (forget gates mostly open in one request, so that the maximum and the memory travel far)
    norm = torch.randn(H * dv, generator=g, dtype=torch.float32)
    eye = torch.eye(width + 2 * H, dtype=F)
    at = {"q": (0, H * d), "k": (H * d, 2 * H * d), "v": (2 * H * d, 2 * H * d + H * dv), "g": (2 * H * d + H * dv, width), "i": (width, width + H), "f": (width + H, width + 2 * H)}
    W = {n: eye[a:b] for n, (a, b) in at.items()}      # (the plain function projects: here every projection picks its columns)
    W.update({"i.b": torch.zeros(H, dtype=F), "f.b": torch.zeros(H, dtype=F), "norm": norm.double(), "o": torch.eye(H * dv, dtype=F)})
    m = {"heads": H, "dim": d, "vdim": dv, "gate_cap": cap}
    want = [pt.mlstm(torch.cat([x, z.double()], 1), W, m, eps) for x, z in zip(raw, zs)]
    state, top = torch.zeros(3, H, d, dv + 1, device=DEV), torch.zeros(3, H, device=DEV)
    got = [torch.zeros(n, H * dv, dtype=F) for n in lengths]
    plans = [cuts(290, (1, 33, 1, 2, 70, 128, 64)), cuts(41, (1, 7, 1, 30, 1))]
    for step in range(max(len(p) for p in plans)):
        live = [(r, *plans[r][step]) for r in range(2) if step < len(plans[r])]
        rows = rows_of([(2 - r, b - a) for r, a, b in live], 3)
        x = torch.cat([raw[r][a:b] for r, a, b in live]).to(dtype).to(DEV).contiguous()
        z = torch.cat([zs[r][a:b] for r, a, b in live]).to(DEV).contiguous()
        T = x.shape[0]
        gates = torch.empty(3, T, H, device=DEV)
        ops.gate_scan(gates, z, top, rows, H, cap)
        qf, kf, vf, dec = (torch.empty(T, H * d, device=DEV), torch.empty(T, H * d, device=DEV), torch.empty(T, H * (dv + 1), device=DEV), torch.empty(T, H * d, device=DEV))
        ops.gated_operands(qf, kf, vf, dec, x[:, :H * d], x[:, H * d:2 * H * d], x[:, 2 * H * d:2 * H * d + H * dv], gates, H, d, dv)
        o = torch.empty(ops.recurrence_max_parts(d), T, H * (dv + 1), device=DEV)
        parts = ops.linear_recurrence(o, qf, kf, vf, state, rows, H, d, dv + 1, ops.DECAY_GIVEN, dec, q_scale=d ** -0.5)
        y = torch.empty(T, H * dv, dtype=dtype, device=DEV)
        ops.headnorm_gate(y, o, x[:, 2 * H * d + H * dv:], norm.to(DEV), H, dv, eps, exact, parts=parts, gate_kind="sigmoid", extra=1, floor=gates[2])
        k = 0
        for r, a, b in live:
            got[r][a:b] = y[k:k + b - a].double().cpu()
            k += b - a
    for r in range(2):
        err = (got[r] - want[r]).abs().max().item()
        assert err <= (3e-5 if exact else 3e-2) * max(1.0, want[r].abs().max().item()), f"request {r}: {err}"


def test_the_norm_that_adds_and_the_row_handed_on():
    from alofa_amd import ops
    rng = np.random.default_rng(1)
    for width in (48, 1000):
        x, res, w, b = rng.normal(2.0, 3.0, (9, width)), rng.normal(0, 1, (9, width)), rng.normal(1, 0.2, width), rng.normal(0, 0.5, width)
        f32 = lambda a: torch.tensor(a, dtype=torch.float32).double()      # noqa: E731
        want = f32(res) + pt.layer_norm(f32(x), f32(w), f32(b), 1e-5)
        for exact in (True, False):
            out = dev(res)
            ops.layernorm_add(out, dev(x), dev(w), dev(b), 1e-5, exact)
            assert (out.cpu().double() - want).abs().max() <= (2e-6 if exact else 2e-5)
        # the norm in front of the next sub-layer in the same launch: the stream as after the sum, and its norm
        w2, b2 = rng.normal(1, 0.2, width), rng.normal(0, 0.5, width)
        for dtype in (torch.float32, torch.bfloat16):
            out, normed = dev(res), torch.empty(9, width, dtype=dtype, device=DEV)
            ops.layernorm_add_norm(out, dev(x), dev(w), dev(b), 1e-5, normed, dev(w2), dev(b2), 1e-6, exact=dtype is torch.float32)
            assert (out.cpu().double() - want).abs().max() <= 2e-5
            after = pt.layer_norm(out.cpu().double(), f32(w2), f32(b2), 1e-6)
            assert (normed.cpu().double() - after).abs().max() <= (1e-5 if dtype is torch.float32 else 3e-2)
            apart = torch.empty(9, width, dtype=dtype, device=DEV)
            ops.layernorm(apart, out, dev(w2), dev(b2), 1e-6, dtype is torch.float32)
            assert torch.equal(apart, normed)      # (the same sums as the two launches one after the other)
        scale = rng.normal(0, 1, 9)
        scale[3] = 0.0
        for dtype in (torch.float32, torch.bfloat16):
            out, rows = dev(res), dev(x, dtype)
            ops.add_row_scaled(out, rows, dev(scale))
            assert (out.cpu().double() - (f32(res) + f32(scale)[:, None] * rows.cpu().double())).abs().max() <= 1e-5


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,dv,parts", [(1, 300, 1), (1, 2048, 3), (2, 2500, 2), (3, 257, 1)])
def test_wide_rows_normed_and_gated(heads, dv, parts, dtype):
    """Heads wider than a wavefront's kernel takes (several heads normed together as one row): against the plain norm, weight and sigmoid gate."""
    from alofa_amd import ops
    g = torch.Generator().manual_seed(dv)
    T, eps, exact = 5, 1e-5, dtype is torch.float32
    o = torch.randn(parts + 1, T, heads * dv, generator=g, dtype=torch.float32)      # (one part more than is added: it must not be read)
    gate = torch.randn(T, heads * dv, generator=g, dtype=torch.float32).to(dtype)
    w = torch.randn(heads * dv, generator=g, dtype=torch.float32)
    rows = o[:parts].double().sum(0).view(T, heads, dv)
    want = (pt.unit_rms(rows, eps).reshape(T, heads * dv) * w.double()) * torch.sigmoid(gate.double())
    out = torch.empty(T, heads * dv, dtype=dtype, device=DEV)
    ops.headnorm_gate(out, o.to(DEV), gate.to(DEV), w.to(DEV), heads, dv, eps, exact, parts=parts, gate_kind="sigmoid")
    assert (out.double().cpu() - want).abs().max() <= (2e-5 if exact else 3e-2) * max(1.0, want.abs().max().item())

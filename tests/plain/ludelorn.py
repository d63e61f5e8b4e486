"""A plain, slow Ludelorn: whole sequences, float64, no cache, no state carried, one function per mechanism. It shares
nothing with the engine; the tests compare the engine's logits (and its residual stream, layer by layer) with it.

``weights``: name -> torch tensor (any dtype; floats are widened to float64). ``cfg``: the config.json dict.
``store``: optional function applied to what a bfloat16 engine keeps rounded between kernels (see ``rounder``)."""
from __future__ import annotations

import math

import torch

F = torch.float64


def rounder(dtype):
    """x -> x rounded to ``dtype`` and widened again."""
    return lambda x: x.to(dtype).to(F)


def _id(x):
    return x


def rms(x, eps):
    """x over its root mean square along the last axis, eps inside the root."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


# ---------------------------------------------------------------- positions

def frequencies(rot: dict):
    """(one frequency per pair as float32, the factor on cos and sin). With ``scaling`` the frequencies of slow pairs are
    divided by the factor, those of fast pairs stay, a ramp in between; cos and sin grow by 0.1 ln(factor) + 1."""
    n, base = rot["dims"], rot["base"]
    f = [base ** (-2.0 * i / n) for i in range(n // 2)]
    mag = 1.0
    sc = rot.get("scaling")
    if sc is not None:
        def dim_of(turns):
            return n * math.log(sc["original"] / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
        lo = max(math.floor(dim_of(sc["fast"])), 0)
        hi = min(math.ceil(dim_of(sc["slow"])), n - 1)
        for i in range(n // 2):
            ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
            f[i] = f[i] / sc["factor"] * ramp + f[i] * (1.0 - ramp)
        mag = 0.1 * math.log(sc["factor"]) + 1.0
    return torch.tensor(f, dtype=F).to(torch.float32), mag


def angles(pos, rot):
    """cos and sin [T, 1, pairs] in float64 of angles that are formed as 32-bit numbers (position times frequency)."""
    f, mag = frequencies(rot)
    a = (pos.to(torch.float32)[:, None, None] * f[None, None, :]).to(F)
    return torch.cos(a) * mag, torch.sin(a) * mag


def turn_halves(x, pos, rot):
    """x [T, heads, d]: channel i < dims/2 pairs with i + dims/2; the channels from dims on pass."""
    n = rot["dims"]
    c, s = angles(pos, rot)
    u, v = x[..., :n // 2], x[..., n // 2:n]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., n:]], dim=-1)


def turn_neighbours(x, pos, rot):
    """x [T, heads, d]: channel 2i pairs with 2i + 1, for i < dims/2; the channels from dims on pass."""
    n = rot["dims"]
    c, s = angles(pos, rot)
    u, v = x[..., 0:n:2], x[..., 1:n:2]
    turned = torch.stack([u * c - v * s, v * c + u * s], dim=-1).flatten(-2)
    return torch.cat([turned, x[..., n:]], dim=-1)


# ---------------------------------------------------------------- attention

def softmax_rows(scores, seen, sink=None):
    """Softmax along the last axis over the entries ``seen``; ``sink`` [heads]: one more term exp(sink) in every
    denominator of its head (scores [heads, rows, keys])."""
    scores = scores.masked_fill(~seen, float("-inf"))
    top = scores.max(-1, keepdim=True).values
    if sink is not None:
        top = torch.maximum(top, sink[:, None, None])
    e = torch.exp(scores - top)
    total = e.sum(-1, keepdim=True)
    if sink is not None:
        total = total + torch.exp(sink[:, None, None] - top)
    return e / total


def window_mask(T, size):
    i, j = torch.arange(T)[:, None], torch.arange(T)[None, :]
    return (j <= i) & (i - j < size)


def windowed_attention(h, W, m, eps, store=_id):
    """The left branch of a parallel layer: a weighted RMS norm of every query and key head (one weight vector for all
    heads), half-split rotation with stretched frequencies, a window, a sigmoid gate per channel."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = torch.arange(T)
    q = store(h @ W["q"].to(F).T).view(T, H, d)
    k = store(h @ W["k"].to(F).T).view(T, G, d)
    v = store(h @ W["v"].to(F).T).view(T, G, dv)
    q = store(turn_halves(rms(q, eps) * W["q.norm"].to(F), pos, m["rot"]))
    k = store(turn_halves(rms(k, eps) * W["k.norm"].to(F), pos, m["rot"]))
    per = H // G
    scores = torch.einsum("ihc,jhc->hij", q, k.repeat_interleave(per, dim=1)) * m["scale"]
    p = softmax_rows(scores, window_mask(T, m["mask"]["size"])[None])
    o = torch.einsum("hij,jhc->ihc", p, v.repeat_interleave(per, dim=1)).reshape(T, H * dv)
    gate = torch.sigmoid(store(h @ W["g"].to(F).T))
    return store(o * gate) @ W["o"].to(F).T


def pooled_attention(h, W, m, eps, store=_id):
    """The mixer "attention": RMS norm over the whole query and key projections, rotation of neighbouring channels, a window,
    and behind the window one mean key and mean value per whole block of ``pool`` tokens (where the layer has blocks); tokens and
    blocks in one softmax."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    size = m["mask"]["size"]
    P = m["mask"].get("pool") or T + 1      # (no blocks: none is ever whole)
    pos = torch.arange(T)
    q = rms(store(h @ W["q"].to(F).T), eps) * W["q.norm"].to(F)
    k = rms(store(h @ W["k"].to(F).T), eps) * W["k.norm"].to(F)
    v = store(h @ W["v"].to(F).T).view(T, G, dv)
    q = store(turn_neighbours(q.view(T, H, d), pos, m["rot"]))
    k = store(turn_neighbours(k.view(T, G, d), pos, m["rot"]))
    nb = T // P
    bk = store(k[:nb * P].view(nb, P, G, d).mean(1))
    bv = store(v[:nb * P].view(nb, P, G, dv).mean(1))
    per = H // G
    s_tok = torch.einsum("ihc,jhc->hij", q, k.repeat_interleave(per, dim=1)) * m["scale"]
    s_blk = torch.einsum("ihc,bhc->hib", q, bk.repeat_interleave(per, dim=1)) * m["scale"]
    last = torch.arange(nb)[None, :] * P + P - 1
    seen_blk = last <= pos[:, None] - size
    p = softmax_rows(torch.cat([s_tok, s_blk], dim=-1), torch.cat([window_mask(T, size), seen_blk], dim=-1)[None])
    o = (torch.einsum("hij,jhc->ihc", p[..., :T], v.repeat_interleave(per, dim=1))
         + torch.einsum("hib,bhc->ihc", p[..., T:], bv.repeat_interleave(per, dim=1))).reshape(T, H * dv)
    gate = torch.sigmoid(store(h @ W["g"].to(F).T))
    return store(o * gate) @ W["o"].to(F).T


def distance_bucket(n: int, rows: int, far: float) -> int:
    """The row of the bias table for distance n: one row per distance up to half the table, then rows spaced evenly in
    the logarithm of the distance up to ``far``."""
    half = rows // 2
    if n < half:
        return n
    return min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (rows - half))))


def biased_attention(h, W, m, eps, store=_id):
    """The mixer "attention_2": values are the keys as projected; queries and keys over their root mean square, no
    positions but a learned bias by distance; a window; a sink in every head's denominator; one gate per head."""
    T = h.shape[0]
    H, G, d = m["heads"], m["kv_heads"], m["dim"]
    size = m["mask"]["size"]
    q = store(h @ W["q"].to(F).T).view(T, H, d)
    kv = store(h @ W["k"].to(F).T).view(T, G, d)
    q, k = store(rms(q, eps)), store(rms(kv, eps))
    per = H // G
    scores = torch.einsum("ihc,jhc->hij", q, k.repeat_interleave(per, dim=1)) * m["scale"]
    rel = W["rel"].to(F)
    rows = rel.shape[0]
    i, j = torch.arange(T)[:, None], torch.arange(T)[None, :]
    buckets = torch.tensor([distance_bucket(n, rows, m["bias_max"]) for n in range(T)])
    bias = rel[buckets[(i - j).clamp(min=0)]]                     # [T, T, H]
    scores = scores + bias.permute(2, 0, 1)
    p = softmax_rows(scores, window_mask(T, size)[None], sink=W["sink"].to(F))
    o = torch.einsum("hij,jhc->ihc", p, kv.repeat_interleave(per, dim=1))
    gate = torch.sigmoid(store(h @ W["g"].to(F).T))               # [T, H]
    return store(o * gate[:, :, None]).reshape(T, H * d) @ W["o"].to(F).T


# ---------------------------------------------------------------- state space

def causal_conv(x, w, b):
    """y_t = b + sum_j w[:, j] x_(t - taps + 1 + j) per channel, zeros before the start. x [T, C], w [C, taps]."""
    T, taps = x.shape[0], w.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, x.shape[1], dtype=F), x])
    return b + sum(padded[j:j + T] * w[:, j] for j in range(taps))


def state_space(h, W, m, eps, store=_id):
    """The right branch of a parallel layer: per head a state S [state, vdim], S_t = exp(-exp(A_log) dt_t) S_(t-1) + dt_t B_t x_t^T,
    y_t = S_t^T C_t + D x_t; B and C shared by the heads of a group; x, B, C through a short convolution and silu;
    y times silu(z), RMS norm in equal parts, output projection."""
    T = h.shape[0]
    H, dv, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = H * dv
    proj = store(h @ W["in"].to(F).T)
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * G * N], proj[:, 2 * inner + 2 * G * N:]
    xbc = store(silu(causal_conv(xbc, W["conv"].to(F), W["conv.b"].to(F))))
    x = xbc[:, :inner].view(T, H, dv)
    B = xbc[:, inner:inner + G * N].view(T, G, N).repeat_interleave(H // G, dim=1)
    C = xbc[:, inner + G * N:].view(T, G, N).repeat_interleave(H // G, dim=1)
    dt = softplus(dt + W["dt_bias"].to(F))
    decay = torch.exp(-torch.exp(W["A_log"].to(F)) * dt)           # [T, H]
    S = torch.zeros(H, N, dv, dtype=F)
    y = torch.zeros(T, H, dv, dtype=F)
    for t in range(T):
        S = decay[t, :, None, None] * S + dt[t, :, None, None] * B[t, :, :, None] * x[t, :, None, :]
        y[t] = torch.einsum("hnv,hn->hv", S, C[t]) + W["D"].to(F)[:, None] * x[t]
    y = y.reshape(T, inner) * silu(z)
    parts = m["norm_groups"]
    y = rms(y.view(T, parts, inner // parts), eps).reshape(T, inner) * W["norm"].to(F)
    return store(y) @ W["o"].to(F).T


def sub(W, prefix):
    return {k[len(prefix):]: v for k, v in W.items() if k.startswith(prefix)}


def parallel(h, W, m, eps, store=_id):
    """Half the sum of the two branches, each through an RMS norm over the width with its weight."""
    left = windowed_attention(h, sub(W, "left."), m["left"], eps, store)
    right = state_space(h, sub(W, "right."), m["right"], eps, store)
    return 0.5 * (rms(left, eps) * W["left.out"].to(F) + rms(right, eps) * W["right.out"].to(F))


# ---------------------------------------------------------------- the model

def dense(h, W, store=_id):
    a = store(gelu_tanh(store(h @ W["up"].to(F).T + W["up.b"].to(F))))
    return a @ W["down"].to(F).T + W["down.b"].to(F)


MIXERS = {"parallel": parallel, "attention": pooled_attention, "attention_2": biased_attention}


def forward(cfg, weights, tokens, store=_id, layers_out=None):
    """Logits [T, vocab] of one sequence. ``layers_out``: a list that receives the stream after every layer."""
    eps = cfg["norm"]["eps"]
    x = weights["embed"].to(F)[torch.tensor(tokens)] * cfg["embedding"]["scale"]
    for i, l in enumerate(cfg["layers"]):
        W = sub(weights, f"l{i}.")
        h = store(rms(x, eps) * W["norm1"].to(F))
        x = x + W["ls1"].to(F) * MIXERS[l["type"]](h, sub(W, "mix."), l["mixer"], eps, store)
        if l.get("mlp") is not None:
            h = store(rms(x, eps) * W["norm2"].to(F))
            x = x + W["ls2"].to(F) * dense(h, sub(W, "mlp."), store)
        if layers_out is not None:
            layers_out.append(x.clone())
    return store(rms(x, eps) * weights["final.norm"].to(F)) @ weights["head"].to(F).T


# ---------------------------------------------------------------- for the tests

def read_config(model_dir):
    import json
    from pathlib import Path
    return json.loads((Path(model_dir) / "config.json").read_text())


def read_weights(model_dir):
    from pathlib import Path
    from safetensors.torch import load_file
    return {k: v.to(F) for k, v in load_file(str(Path(model_dir) / "model.safetensors")).items()}


def to_bfloat16(x):
    return x.to(torch.bfloat16).to(F)


def forward_logits(weights, cfg, tokens, store=_id):
    return forward(cfg, weights, tokens, store).numpy()


def forward_hidden(weights, cfg, tokens):
    out = []
    forward(cfg, weights, tokens, layers_out=out)
    return [x.numpy() for x in out]


def greedy(weights, cfg, prompt, n_new):
    ids = list(prompt)
    for _ in range(n_new):
        ids.append(int(forward(cfg, weights, ids)[-1].argmax()))
    return ids[len(prompt):]

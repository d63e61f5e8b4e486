"""A plain, slow Retotar: whole sequences, float64, no cache, no state, one function per mechanism. It shares
nothing with the engine; the tests compare the engine's logits (and its residual stream, layer by layer) with it.

``weights``: name -> torch tensor (any float dtype; everything is widened to float64). ``cfg``: the config.json dict.
``store``: optional function applied to what a bfloat16 engine keeps rounded between kernels (see ``rounder``)."""
from __future__ import annotations

import torch

F = torch.float64


def rounder(dtype):
    """x -> x rounded to ``dtype`` and widened again."""
    return lambda x: x.to(dtype).to(F)


def _id(x):
    return x


def layer_norm(x, w, b, eps):
    mean = x.mean(-1, keepdim=True)
    var = ((x - mean) ** 2).mean(-1, keepdim=True)
    return (x - mean) / torch.sqrt(var + eps) * w + b


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def silu(z):
    return z * torch.sigmoid(z)


def turn_halves(x, pos, n, base, factor=1.0, sign=1.0):
    """The first ``n`` channels of the last axis turned by the positions' angles: channel i pairs with i + n/2, the angle
    of pair i is pos * base^(-2i/n) / factor; the rest passes. x [T, heads, d], pos [T]."""
    half = n // 2
    # (frequencies and angles are 32-bit numbers in this design: the angle of a far position is known to some 1e-5 only, and a twin that
    # knew it better would differ from every engine by that much)
    f = torch.tensor(1.0, dtype=torch.float32) / torch.tensor([base ** (2.0 * i / n) for i in range(half)], dtype=F).to(torch.float32)
    if factor != 1.0:
        f = f / torch.tensor(factor, dtype=torch.float32)
    a = sign * (pos.to(torch.float32)[:, None, None] * f[None, None, :]).to(F)
    u, v = x[..., :half], x[..., half:n]
    return torch.cat([u * torch.cos(a) - v * torch.sin(a), v * torch.cos(a) + u * torch.sin(a), x[..., n:]], dim=-1)


def attention_keys_values(h, W, m, eps, store=_id):
    """(keys after rotation and unit norm, values after their rotation) of a layer with projections: [T, G, dim], [T, G, vdim]."""
    T = h.shape[0]
    G, d, dv = m["kv_heads"], m["dim"], m["vdim"]
    rot = m["rot"]
    factor = (rot.get("scaling") or {}).get("factor", 1.0)
    pos = torch.arange(T)
    k = store(h @ W["k"].to(F).T).view(T, G, d)
    v = store(h @ W["v"].to(F).T).view(T, G, dv)
    k = unit_rms(turn_halves(k, pos, rot["dims"], rot["base"], factor), eps)
    v = turn_halves(v, pos, dv, rot["base"])
    return store(k), store(v)


def attention(h, W, m, eps, keys_values=None, store=_id):
    """Softmax attention within a window, the heads' weights mixed after the softmax, values turned by their positions and the
    result turned back, a sigmoid gate. ``keys_values``: another layer's (a layer with ``kv_from``)."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    rot = m["rot"]
    factor = (rot.get("scaling") or {}).get("factor", 1.0)
    pos = torch.arange(T)
    q = store(h @ W["q"].to(F).T).view(T, H, d)
    q = unit_rms(turn_halves(q, pos, rot["dims"], rot["base"], factor), eps)
    k, v = keys_values if keys_values is not None else attention_keys_values(h, W, m, eps, store)
    per = H // G
    scores = torch.einsum("ihc,jhc->hij", q, k.repeat_interleave(per, dim=1)) * m["scale"]
    i, j = pos[:, None], pos[None, :]
    seen = (j <= i)
    if m.get("mask") is not None:
        seen = seen & (i - j < m["mask"]["size"])
    scores = scores.masked_fill(~seen[None], float("-inf"))
    p = torch.softmax(scores, dim=-1)
    p = torch.einsum("hg,gij->hij", W["talk"].to(F), p)
    o = torch.einsum("hij,jhc->ihc", p, v.repeat_interleave(per, dim=1))
    o = turn_halves(o, pos, dv, rot["base"], sign=-1.0)
    gate = torch.sigmoid(store(h @ W["g"].to(F).T))
    return store(o.reshape(T, H * dv) * gate) @ W["o"].to(F).T


def lightning(h, W, m, eps, store=_id):
    """S_t = decay S_(t-1) + k_t v_t^T per head, o_t = S_t^T q_t; q, k, v through silu; the heads together through an RMS norm
    with a weight, a sigmoid gate, the output projection."""
    T = h.shape[0]
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    q = store(silu(store(h @ W["q"].to(F).T))).view(T, H, d)
    k = store(silu(store(h @ W["k"].to(F).T))).view(T, H, d)
    v = store(silu(store(h @ W["v"].to(F).T))).view(T, H, dv)
    decay = torch.tensor(m["decay"], dtype=F)
    S = torch.zeros(H, d, dv, dtype=F)
    o = torch.zeros(T, H, dv, dtype=F)
    for t in range(T):
        S = decay[:, None, None] * S + k[t, :, :, None] * v[t, :, None, :]
        o[t] = torch.einsum("hkv,hk->hv", S, q[t])
    y = unit_rms(o.reshape(T, H * dv), eps) * W["norm"].to(F)
    gate = torch.sigmoid(store(h @ W["g"].to(F).T))
    return store(y * gate) @ W["o"].to(F).T


def mlstm(h, W, m, eps, store=_id):
    """A matrix memory with exponential gates kept in range by a running maximum that starts at zero."""
    T = h.shape[0]
    H, d, dv, cap = m["heads"], m["dim"], m["vdim"], m["gate_cap"]
    q = store(h @ W["q"].to(F).T).view(T, H, d) * d ** -0.5
    k = store(h @ W["k"].to(F).T).view(T, H, d)
    v = store(h @ W["v"].to(F).T).view(T, H, dv)
    gi = cap * torch.tanh((h @ W["i"].to(F).T + W["i.b"].to(F)) / cap)
    gf = torch.nn.functional.logsigmoid(cap * torch.tanh((h @ W["f"].to(F).T + W["f.b"].to(F)) / cap))
    S = torch.zeros(H, d, dv, dtype=F)
    n = torch.zeros(H, d, dtype=F)
    mx = torch.zeros(H, dtype=F)
    o = torch.zeros(T, H, dv, dtype=F)
    for t in range(T):
        new = torch.maximum(gf[t] + mx, gi[t])
        keep, take = torch.exp(gf[t] + mx - new), torch.exp(gi[t] - new)
        S = keep[:, None, None] * S + take[:, None, None] * k[t, :, :, None] * v[t, :, None, :]
        n = keep[:, None] * n + take[:, None] * k[t]
        mx = new
        den = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-mx)) + 1e-6
        o[t] = torch.einsum("hkv,hk->hv", S, q[t]) / den[:, None]
    y = unit_rms(o, eps).reshape(T, H * dv) * W["norm"].to(F)
    gate = torch.sigmoid(store(h @ W["g"].to(F).T))
    return store(y * gate) @ W["o"].to(F).T


def choose_experts(z, correction, r):
    """(chosen [T, top], weights [T, top]) from router products z [T, E + identity]."""
    E_all = z.shape[1]
    s = torch.softmax(z, dim=-1)
    c = s + correction
    groups = r.get("groups") or {"count": 1, "keep": 1}
    size = E_all // groups["count"]
    best = c.view(-1, groups["count"], size).max(-1).values
    kept = torch.topk(best, groups["keep"], dim=-1).indices
    allowed = torch.zeros_like(best, dtype=torch.bool).scatter_(1, kept, True).repeat_interleave(size, dim=1)
    c = c.masked_fill(~allowed, float("-inf"))
    chosen = torch.topk(c, r["top"], dim=-1).indices
    return chosen, torch.gather(s, 1, chosen)


def experts(h, W, mlp, store=_id):
    """A mixture of gated feed-forwards; the last ``identity`` router outputs stand for experts that hand the input on."""
    r = mlp["router"]
    E, ident = r["experts"], r.get("identity", 0)
    z = h @ W["router"].to(F).T
    chosen, weights = choose_experts(z, W["correction"].to(F), r)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, w in zip(chosen[t].tolist(), weights[t]):
            if e >= E:
                out[t] += w * h[t]
                continue
            a = store(silu(h[t] @ W[f"e{e}.gate"].to(F).T) * (h[t] @ W[f"e{e}.up"].to(F).T))
            out[t] += w * (a @ W[f"e{e}.down"].to(F).T)
    assert ident >= 0
    return out


def _sub(weights, prefix):
    return {k[len(prefix):]: v for k, v in weights.items() if k.startswith(prefix)}


def forward(cfg, weights, tokens, store=_id, layers_out=None):
    """Logits [T, vocab] (float64) of one sequence. ``layers_out``: a list that receives the stream after every layer."""
    eps = cfg["norm"]["eps"]
    ids = torch.as_tensor(tokens, dtype=torch.long)
    x = weights["embed"].to(F)[ids] * cfg["embedding"]["scale"]
    kept = {}

    def norm(name, v):
        return layer_norm(v, weights[name].to(F), weights[name + ".b"].to(F), eps)

    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        W = _sub(weights, p + "mix.")
        h = store(norm(p + "norm1", x))
        if layer["type"] == "attention":
            if m.get("kv_from") is not None:
                y = attention(h, W, m, eps, kept[m["kv_from"]], store)
            else:
                kept[i] = attention_keys_values(h, W, m, eps, store)
                y = attention(h, W, m, eps, kept[i], store)
        elif layer["type"] == "lightning":
            y = lightning(h, W, m, eps, store)
        elif layer["type"] == "mlstm":
            y = mlstm(h, W, m, eps, store)
        else:
            raise ValueError(layer["type"])
        x = x + norm(p + "norm1b", y)
        if layer.get("mlp") is not None:
            h = store(norm(p + "norm2", x))
            x = x + norm(p + "norm2b", experts(h, _sub(weights, p + "mlp."), layer["mlp"], store))
        if layers_out is not None:
            layers_out.append(x.clone())
    y = store(norm("final.norm", x))
    return y @ weights["head"].to(F).T


# ---- for the tests: folders, logits as arrays, how close the routers' calls are, greedy continuation

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


def router_margins(weights, cfg, tokens):
    """Per position the smallest gap, over all layers, between what a router takes and what it leaves (experts and groups), relative to
    the scores that a change of the router's input would move."""
    eps = cfg["norm"]["eps"]
    T = len(tokens)
    margins = torch.full((T,), float("inf"), dtype=F)
    seen = []
    forward(cfg, weights, tokens, layers_out=seen)
    ids = torch.as_tensor(tokens, dtype=torch.long)
    x0 = weights["embed"].to(F)[ids] * cfg["embedding"]["scale"]
    for i, layer in enumerate(cfg["layers"]):
        if layer.get("mlp") is None:
            continue
        # the stream in front of the feed-forward: the layer's output minus what the feed-forward added is not kept, so it is made again
        p = f"l{i}."
        before = x0 if i == 0 else seen[i - 1]
        W = _sub(weights, p + "mix.")
        h = layer_norm(before, weights[p + "norm1"].to(F), weights[p + "norm1.b"].to(F), eps)
        m = layer["mixer"]
        if layer["type"] == "attention":
            src = m.get("kv_from")
            if src is None:
                kv = attention_keys_values(h, W, m, eps)
            else:
                prev = x0 if src == 0 else seen[src - 1]
                hs = layer_norm(prev, weights[f"l{src}.norm1"].to(F), weights[f"l{src}.norm1.b"].to(F), eps)
                kv = attention_keys_values(hs, _sub(weights, f"l{src}.mix."), cfg["layers"][src]["mixer"], eps)
            y = attention(h, W, m, eps, kv)
        elif layer["type"] == "lightning":
            y = lightning(h, W, m, eps)
        else:
            y = mlstm(h, W, m, eps)
        x = before + layer_norm(y, weights[p + "norm1b"].to(F), weights[p + "norm1b.b"].to(F), eps)
        h2 = layer_norm(x, weights[p + "norm2"].to(F), weights[p + "norm2.b"].to(F), eps)
        r = layer["mlp"]["router"]
        Wm = _sub(weights, p + "mlp.")
        s = torch.softmax(h2 @ Wm["router"].to(F).T, dim=-1)
        c = s + Wm["correction"].to(F)
        groups = r.get("groups") or {"count": 1, "keep": 1}
        size = c.shape[1] // groups["count"]
        best = c.view(T, groups["count"], size).max(-1).values
        # a gap between two choice scores counts against the softmax scores behind them: those are what a small change of z moves
        order = best.sort(-1, descending=True)
        if groups["keep"] < groups["count"]:
            at = c.view(T, groups["count"], size).argmax(-1) + torch.arange(groups["count"]) * size      # the member behind a group's score
            s_best = torch.gather(torch.gather(s, 1, at), 1, order.indices)
            gap = order.values[:, groups["keep"] - 1] - order.values[:, groups["keep"]]
            margins = torch.minimum(margins, gap / (s_best[:, groups["keep"] - 1] + s_best[:, groups["keep"]]))
        kept = order.indices[:, :groups["keep"]]
        allowed = torch.zeros_like(best, dtype=torch.bool).scatter_(1, kept, True).repeat_interleave(size, dim=1)
        ca = c.masked_fill(~allowed, float("-inf")).sort(-1, descending=True)
        if r["top"] < int(allowed[0].sum()):
            sa = torch.gather(s, 1, ca.indices)
            gap = ca.values[:, r["top"] - 1] - ca.values[:, r["top"]]
            margins = torch.minimum(margins, gap / (sa[:, r["top"] - 1] + sa[:, r["top"]]))
    return margins.numpy()


def greedy(weights, cfg, prompt, n_new):
    ids = list(prompt)
    for _ in range(n_new):
        ids.append(int(forward(cfg, weights, ids)[-1].argmax()))
    return ids[len(prompt):]

"""Ludelorn without a GPU: the configuration's keys and checks, the tensor list, sizes taken from tensors' shapes, what every layer keeps
per token and per request, the tables of angles and of bias rows against the plain implementation, and the plain implementation's own
consistency."""
import copy
import json
import math

import numpy as np
import pytest
import torch

from alofa_amd.config.base import PartSpec
from alofa_amd.config.registry import config_from_dict, load_config
from alofa_amd.errors import AlofaError
from alofa_amd.model import check_spec, expected_tensors
from alofa_amd.weights import write_random_model
from ludelorn_cases import LUDELORN
from plain import ludelorn as pl


@pytest.mark.parametrize("name", list(LUDELORN))
def test_config_round_trip_and_tensor_list(name, tmp_path):
    cfg = config_from_dict(LUDELORN[name])
    assert config_from_dict(cfg.to_dict()) == cfg
    spec = cfg.spec()
    check_spec(spec)
    write_random_model(LUDELORN[name], tmp_path, seed=1)
    assert load_config(tmp_path) == cfg
    w = pl.read_weights(tmp_path)
    expected = expected_tensors(spec)
    assert set(w) == {n for n, r in expected.items() if not r.optional}
    assert all(tuple(w[n].shape) == tuple(expected[n].shape) for n in w)
    assert w["final.norm"].shape == () and w["l0.norm1"].shape == ()
    for i, l in enumerate(LUDELORN[name]["layers"]):
        p = f"l{i}."
        assert (p + "mix.left.out" in w) == (p + "mix.right.conv.b" in w) == (l["type"] == "parallel")
        assert (p + "mix.rel" in w) == (p + "mix.sink" in w) == (l["type"] == "attention_2")
        assert (p + "mix.v" in w) == (l["type"] == "attention")
        assert (p + "norm2" in w) == (p + "ls2" in w) == (p + "mlp.down.b" in w) == (l["mlp"] is not None)
        if l["type"] == "attention_2":
            assert tuple(w[p + "mix.g"].shape) == (l["mixer"]["heads"], LUDELORN[name]["width"])
            assert tuple(w[p + "mix.rel"].shape) == (l["mixer"]["bias_rows"], l["mixer"]["heads"])
        if l["type"] == "attention":
            assert w[p + "mix.q.norm"].shape[0] == l["mixer"]["heads"] * l["mixer"]["dim"]
        if l["type"] == "parallel":
            r = l["mixer"]["right"]
            assert w[p + "mix.right.in"].shape[0] == 2 * r["heads"] * r["vdim"] + 2 * r["groups"] * r["state"] + r["heads"]
            assert w[p + "mix.left.q.norm"].shape[0] == l["mixer"]["left"]["dim"]


def test_the_bias_table_is_sized_by_its_tensor(tmp_path):
    write_random_model(LUDELORN["A"], tmp_path, seed=1)
    raw = json.loads((tmp_path / "config.json").read_text())
    for l in raw["layers"]:
        l["mixer"].pop("bias_rows", None)
    bare = config_from_dict(raw)
    assert bare.wants_shapes()
    with pytest.raises(AlofaError, match="rows of a bias table"):
        bare.spec()
    (tmp_path / "config.json").write_text(json.dumps(raw))
    assert load_config(tmp_path) == config_from_dict(LUDELORN["A"])


@pytest.mark.parametrize("change, message", [
    (lambda c: c["layers"][0].update(type="windowed"), "no such mixer"),
    (lambda c: c["layers"][0]["mlp"].update(kind="moe"), "no such feed-forward"),
    (lambda c: c["layers"][0]["mixer"]["left"].update(kv_heads=3), "kv_heads must divide heads"),
    (lambda c: c["layers"][0]["mixer"]["left"]["rot"].update(dims=18), "rot.dims is even and at most"),
    (lambda c: c["layers"][0]["mixer"]["right"].update(groups=3), "groups divide the heads"),
    (lambda c: c["layers"][0]["mixer"]["right"].update(norm_groups=5), "groups divide the heads"),
    (lambda c: c["layers"][1]["mixer"]["mask"].update(pool=0), "must be positive"),
    (lambda c: c["layers"][2]["mixer"].update(vdim=8), "values that are the keys"),
    (lambda c: c["layers"][2]["mixer"].pop("bias_max"), "lacks a required key"),
    (lambda c: c.update(layers=[]), "at least one layer"),
])
def test_config_checks(change, message):
    cfg = copy.deepcopy(LUDELORN["A"])
    change(cfg)
    with pytest.raises(AlofaError, match=message):
        config_from_dict(cfg).spec()


def test_what_every_layer_keeps():
    """Pages by window (a pooled layer keeps its window's pages at least as long as a block, and its blocks for good), state per request."""
    from alofa_amd.parts.base import part_class, SLOT
    from alofa_amd.parts.base import CacheTensor
    spec = config_from_dict(LUDELORN["B"]).spec()
    pooled = spec.layers[1].parts["mixer"].params
    assert (pooled["window"], pooled["pool"]) == (9, 16)
    assert CacheTensor("pk", (2, SLOT, 8), every=5).page_shape(16) == (2, 4, 8)      # blocks begin at tokens 0, 5, 10, 15 of a page
    assert CacheTensor("pk", (2, SLOT, 8), every=16).page_shape(16) == (2, 1, 8)
    assert CacheTensor("pk", (2, SLOT, 8), every=40).page_shape(16) == (2, 1, 8)
    assert CacheTensor("k", (2, SLOT, 8)).page_shape(16) == (2, 16, 8)
    parallel = spec.layers[2].parts["mixer"]
    assert parallel.kind == "parallel" and parallel.params["scales"] == (0.5, 0.5) and [b.kind for b in parallel.params["branches"]] == ["window_attention", "state_space"]
    assert part_class("mixer", "state_space") is not None and part_class("mixer", "window_attention") is not None


@pytest.mark.parametrize("rot", [
    {"base": 10000.0, "dims": 8, "scaling": {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 2.0}},
    {"base": 250000.0, "dims": 32, "scaling": {"factor": 3.0, "original": 1024, "fast": 16.0, "slow": 2.0}},
    {"base": 777.0, "dims": 6},
    {"base": 50.0, "dims": 16, "scaling": {"factor": 8.0, "original": 16, "fast": 2.0, "slow": 1.5}},
])
@pytest.mark.parametrize("pairing", ["half", "neighbours"])
def test_the_table_of_angles_is_the_plain_one(rot, pairing):
    """cos and sin of the engine's table against the plain frequencies, and the order of channels in which the design's pairs lie as the
    kernels pair them, for heads wider than the turned channels."""
    from alofa_amd.parts.position import Rotary
    d = rot["dims"] + 6
    part = Rotary(PartSpec("rotary", {"theta": rot["base"], "head_dim": d, "dims": rot["dims"], "pairing": pairing, "frequencies": "direct", "stretch": rot.get("scaling")}), {}, None)
    cos, sin = part.host_table(700)
    pos = torch.arange(700)
    c, s = pl.angles(pos, rot)
    half = rot["dims"] // 2
    assert np.abs(cos[:, :half] - c[:, 0].numpy()).max() < 1e-6 and np.abs(sin[:, :half] - s[:, 0].numpy()).max() < 1e-6
    assert (cos[:, half:] == 1.0).all() and (sin[:, half:] == 0.0).all()      # (the channels that are not turned pass as they are)
    # turning a random head by the table in the kernels' pairing, in the part's order of channels, is the plain turn
    x = torch.randn(700, 1, d, dtype=torch.float64)
    want = (pl.turn_halves if pairing == "half" else pl.turn_neighbours)(x, pos, rot)
    order = part.channel_order() or list(range(d))
    y = x[..., order]
    C, S = torch.from_numpy(cos).double()[:, None, :], torch.from_numpy(sin).double()[:, None, :]
    u, v = y[..., :d // 2], y[..., d // 2:]
    turned = torch.cat([u * C - v * S, v * C + u * S], dim=-1)
    back = torch.empty_like(turned)
    back[..., order] = turned
    assert (back - want).abs().max() < 2e-6


def test_the_bias_rows_are_the_plain_ones():
    from alofa_amd.parts.window import distance_buckets
    for rows, far in ((24, 90.0), (8, 14.0), (6, 5.0), (2, 3.0), (16, 30.0), (7, 100.5)):
        upto = int(math.ceil(far)) + 3
        assert distance_buckets(rows, far, upto) == [pl.distance_bucket(n, rows, far) for n in range(upto)]
        assert pl.distance_bucket(10 ** 6, rows, far) == rows - 1 == distance_buckets(rows, far, upto)[-1]


def test_the_plain_model_agrees_with_itself():
    """Two readings of the same equations: the pooled layer with blocks of one token is attention over everything; the state-space
    recurrence is its unrolled sum; a sink of minus infinity is no sink."""
    torch.manual_seed(0)
    T, eps = 40, 1e-5
    m = {"heads": 2, "kv_heads": 1, "dim": 8, "vdim": 6, "rot": {"base": 100.0, "dims": 4}, "scale": 0.3, "mask": {"size": 5, "pool": 1}}
    W = {k: torch.randn(s, dtype=torch.float64) for k, s in (("q", (16, 12)), ("k", (8, 12)), ("v", (6, 12)), ("g", (12, 12)), ("o", (12, 12)), ("q.norm", (16,)), ("k.norm", (8,)))}
    h = torch.randn(T, 12, dtype=torch.float64)
    everything = copy.deepcopy(m)
    everything["mask"] = {"size": T + 1}
    assert (pl.pooled_attention(h, W, m, eps) - pl.pooled_attention(h, W, everything, eps)).abs().max() < 1e-9
    r = {"heads": 2, "vdim": 3, "state": 4, "groups": 1, "conv": 2, "norm_groups": 1}
    Wr = {k: torch.randn(s, dtype=torch.float64) * 0.5 for k, s in (("in", (2 * 6 + 8 + 2, 12)), ("conv", (14, 2)), ("conv.b", (14,)), ("dt_bias", (2,)), ("A_log", (2,)),
                                                                    ("D", (2,)), ("norm", (6,)), ("o", (12, 6)))}
    out = pl.state_space(h, Wr, r, eps)
    proj = h @ Wr["in"].T
    xbc = pl.silu(pl.causal_conv(proj[:, 6:20], Wr["conv"], Wr["conv.b"]))
    x, B, C = xbc[:, :6].view(T, 2, 3), xbc[:, 6:10], xbc[:, 10:14]
    dt = torch.log1p(torch.exp(proj[:, 20:] + Wr["dt_bias"]))
    la = -torch.exp(Wr["A_log"]) * dt
    y = torch.zeros(T, 2, 3, dtype=torch.float64)
    for t in range(T):
        for s in range(t + 1):
            y[t] += torch.exp(la[s + 1:t + 1].sum(0))[:, None] * dt[s][:, None] * (B[s] @ C[t]) * x[s]
        y[t] += Wr["D"][:, None] * x[t]
    y = pl.rms((y.reshape(T, 6) * pl.silu(proj[:, :6])), eps) * Wr["norm"]
    assert (out - y @ Wr["o"].T).abs().max() < 1e-9
    b = {"heads": 2, "kv_heads": 2, "dim": 4, "scale": 0.5, "mask": {"size": 6}, "bias_max": 9.0}
    Wb = {k: torch.randn(s, dtype=torch.float64) for k, s in (("q", (8, 12)), ("k", (8, 12)), ("g", (2, 12)), ("o", (12, 8)), ("rel", (4, 2)))}
    with_sink = pl.biased_attention(h, {**Wb, "sink": torch.tensor([-1e9, -1e9], dtype=torch.float64)}, b, eps)
    zero_sink = pl.biased_attention(h, {**Wb, "sink": torch.zeros(2, dtype=torch.float64)}, b, eps)
    assert (with_sink - zero_sink).abs().max() > 1e-3      # exp(0) in the denominator takes weight away
    first_row = torch.softmax(torch.tensor([0.0]), 0)      # a single key and no sink: weight one
    assert first_row.item() == 1.0

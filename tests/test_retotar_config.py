"""Retotar without a GPU: the configuration's keys and checks, the tensor list, whose pages a layer reads and how long they are
kept, and the plain implementation's own consistency."""
import copy

import numpy as np
import pytest
import torch

from alofa_amd.config.registry import config_from_dict, load_config
from alofa_amd.errors import AlofaError
from alofa_amd.model import check_spec, expected_tensors
from alofa_amd.weights import write_random_model
from plain import retotar as pt
from retotar_cases import RETOTAR


@pytest.mark.parametrize("name", list(RETOTAR))
def test_config_round_trip_and_tensor_list(name, tmp_path):
    cfg = config_from_dict(RETOTAR[name])
    assert config_from_dict(cfg.to_dict()) == cfg
    spec = cfg.spec()
    check_spec(spec)
    write_random_model(RETOTAR[name], tmp_path, seed=1)
    assert load_config(tmp_path) == cfg
    w = pt.read_weights(tmp_path)
    expected = expected_tensors(spec)
    assert set(w) == {n for n, r in expected.items() if not r.optional}
    assert all(tuple(w[n].shape) == tuple(expected[n].shape) for n in w)
    for i, l in enumerate(RETOTAR[name]["layers"]):
        m, p = l["mixer"], f"l{i}."
        assert (p + "mix.k" in w) == (p + "mix.v" in w) == (l["type"] != "attention" or "kv_from" not in m)
        assert (p + "mix.talk" in w) == (l["type"] == "attention") and (p + "mix.i.b" in w) == (l["type"] == "mlstm")
        assert (p + "norm2b.b" in w) == (l["mlp"] is not None)
        if l["mlp"] is not None:
            r = l["mlp"]["router"]
            assert w[p + "mlp.router"].shape[0] == w[p + "mlp.correction"].shape[0] == r["experts"] + r["identity"]
            assert p + f"mlp.e{r['experts'] - 1}.down" in w and p + f"mlp.e{r['experts']}.down" not in w


def test_whose_pages_a_layer_reads_and_how_long_they_are_kept():
    spec = config_from_dict(RETOTAR["A"]).spec()      # layer 3 reads layer 0's pages through a longer window
    assert [e.cache_of for e in spec.order] == [None, None, None, 0]
    first, last = spec.layers[0].parts["mixer"].params, spec.layers[3].parts["mixer"].params
    assert (first["window"], first["keep_window"], first["owns_cache"]) == (20, 33, True)
    assert (last["window"], last["keep_window"], last["owns_cache"]) == (33, 33, False)
    spec = config_from_dict(RETOTAR["D"]).spec()      # the reader's window is the shorter one: the owner's decides
    assert spec.layers[0].parts["mixer"].params["keep_window"] == 100 and spec.order[4].cache_of == 0
    spec = config_from_dict(RETOTAR["C"]).spec()      # no mask: every key is kept
    assert spec.layers[2].parts["mixer"].params["keep_window"] is None and spec.layers[2].parts["mixer"].params["window"] is None


@pytest.mark.parametrize("change, message", [
    (lambda c: c["layers"][0].update(type="windowed"), "no such mixer"),
    (lambda c: c["layers"][0]["mlp"].update(kind="dense"), "no such feed-forward"),
    (lambda c: c["layers"][0]["mlp"]["router"].update(top=5), "equal groups"),
    (lambda c: c["layers"][0]["mlp"]["router"]["groups"].update(count=3), "equal groups"),
    (lambda c: c["layers"][0]["mixer"].update(kv_heads=3), "kv_heads must divide heads"),
    (lambda c: c["layers"][0]["mixer"].update(vdim=23), "vdim is even"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=18), "rot.dims is even and at most"),
    (lambda c: c["layers"][3]["mixer"].update(kv_from=1), "kv_from names an earlier attention layer"),
    (lambda c: c["layers"][3]["mixer"].update(kv_from=3), "kv_from names an earlier attention layer"),
    (lambda c: c["layers"][3]["mixer"].update(vdim=16), "kv_from names an earlier attention layer"),
    (lambda c: c["layers"][1]["mixer"].update(decay=[0.5]), "one decay per head"),
    (lambda c: c["layers"][2]["mixer"].pop("gate_cap"), "lacks a required key"),
    (lambda c: c["norm"].update(eps=0.0), "must be positive"),
])
def test_what_the_configuration_refuses(change, message):
    raw = copy.deepcopy(RETOTAR["A"])
    change(raw)
    with pytest.raises(AlofaError) as e:
        config_from_dict(raw)
    assert message in str(e.value)


def test_the_plain_mechanisms_agree_with_their_definitions():
    """The plain functions against even plainer loops, on small random inputs."""
    g = torch.Generator().manual_seed(3)
    # the choice among experts: groups, the correction in the choice and not in the weights
    z = torch.randn(9, 8, generator=g, dtype=torch.float64)
    corr = torch.randn(8, generator=g, dtype=torch.float64) * 0.2
    chosen, weights = pt.choose_experts(z, corr, {"top": 3, "groups": {"count": 4, "keep": 2}})
    for t in range(9):
        s = torch.softmax(z[t], 0)
        c = s + corr
        best = sorted(range(4), key=lambda k: -max(c[2 * k], c[2 * k + 1]))[:2]
        allowed = sorted((e for e in range(8) if e // 2 in best), key=lambda e: -c[e])[:3]
        assert chosen[t].tolist() == allowed and torch.allclose(weights[t], s[allowed])
    # the memory against a sum over the past written out: with the running maximum m_t, S_t = sum_s exp(i_s + F_t - F_s - m_t) k_s v_s^T
    T, H, d, dv = 7, 2, 4, 6
    m = {"heads": H, "dim": d, "vdim": dv, "gate_cap": 5.0}
    W = {n: torch.randn(s, generator=g, dtype=torch.float64) for n, s in (("q", (H * d, 10)), ("k", (H * d, 10)), ("v", (H * dv, 10)), ("g", (H * dv, 10)), ("o", (10, H * dv)),
                                                                            ("i", (H, 10)), ("f", (H, 10)), ("i.b", (H,)), ("f.b", (H,)), ("norm", (H * dv,)))}
    h = torch.randn(T, 10, generator=g, dtype=torch.float64)
    got = pt.mlstm(h, W, m, 1e-6)
    gi = 5.0 * torch.tanh((h @ W["i"].T + W["i.b"]) / 5.0)
    gf = torch.nn.functional.logsigmoid(5.0 * torch.tanh((h @ W["f"].T + W["f.b"]) / 5.0))
    F = gf.cumsum(0)
    out = torch.zeros(T, H, dv, dtype=torch.float64)
    q, k, v = (h @ W["q"].T).view(T, H, d) * d ** -0.5, (h @ W["k"].T).view(T, H, d), (h @ W["v"].T).view(T, H, dv)
    for t in range(T):
        for a in range(H):
            logw = torch.stack([gi[s, a] + F[t, a] - F[s, a] for s in range(t + 1)])
            mt = torch.maximum(logw.max(), F[t, a])      # (the maximum starts at 0 and decays with the forget gates)
            wts = torch.exp(logw - mt)
            num = sum(wts[s] * (q[t, a] @ k[s, a]) * v[s, a] for s in range(t + 1))
            den = torch.maximum(sum(wts[s] * (q[t, a] @ k[s, a]) for s in range(t + 1)).abs(), torch.exp(-mt)) + 1e-6
            out[t, a] = num / den
    want = (pt.unit_rms(out, 1e-6).reshape(T, H * dv) * W["norm"] * torch.sigmoid(h @ W["g"].T)) @ W["o"].T
    assert torch.allclose(got, want, rtol=1e-9, atol=1e-9)
    # turned values: what a head gives depends on distances only (turn by j, turn back by i = turn by j - i)
    x = torch.randn(5, 1, 8, generator=g, dtype=torch.float64)
    once = pt.turn_halves(pt.turn_halves(x, torch.arange(5), 8, 100.0), torch.arange(5) + 3, 8, 100.0, sign=-1.0)
    assert torch.allclose(once, pt.turn_halves(x, torch.full((5,), -3), 8, 100.0))


def test_bfloat16_rounding_of_the_plain_model_is_small():
    cfg = RETOTAR["B"]
    w = {n: t for n, t in ((n, t.double()) for n, t in __import__("alofa_amd.weights.random_init", fromlist=["random_tensors"]).random_tensors(
        expected_tensors(config_from_dict(cfg).spec()), 5).items())}
    ids = [int(t) for t in np.random.default_rng(0).integers(0, cfg["vocab"], 20)]
    exact, rounded = pt.forward_logits(w, cfg, ids), pt.forward_logits(w, cfg, ids, store=pt.to_bfloat16)
    assert 0 < np.abs(exact - rounded).max() < 0.1 * np.abs(exact).max()

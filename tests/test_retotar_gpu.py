"""Retotar through the engine against the plain implementation, in float32 and bfloat16: whole prompts, the stream after every
layer, every mixer alone, decoding token by token, portions down to two tokens, unequal requests in one batch, slots and pages that
are used again, windows whose edges fall on, before and behind page borders, weights made so that single keys decide, and greedy
generation through the engine's own loop."""
import copy
import json

import numpy as np
import pytest

from helpers import assert_close, bulk_and_tail, collect, mixed, portions, random_ids, whole
from plain import retotar as pt
from retotar_cases import RETOTAR, clear_calls, clear_ids, plain_logits, plain_model

pytestmark = pytest.mark.gpu

DTYPES = ["float32", "bfloat16"]
LENGTHS = {"A": 100, "B": 75, "C": 120, "D": 150, "E": 90, "F": 140}


@pytest.fixture(scope="module")
def replayers(retotar_dirs):
    from alofa_amd.replay import Replayer
    made = {}

    def get(name, dtype, max_tokens=512):
        key = (name, dtype, max_tokens)
        if key not in made:
            made[key] = Replayer(retotar_dirs[name], dtype, max_tokens, max_requests=4)
        r = made[key]
        assert not r.cache.requests, "a test left requests behind"
        return r
    return get


def ids_of(dirs, name, n=None):
    return clear_ids(str(dirs[name]), n or LENGTHS[name])


def compare(got, model_dir, ids, dtype, what, least=8):
    rows = clear_calls(model_dir, ids, dtype)
    assert len(rows) >= least, f"{what}: too few positions are left to compare ({len(rows)} of {len(ids)})"
    assert_close(np.asarray(got)[rows], plain_logits(model_dir, tuple(ids))[rows], dtype, what)


def compare_together(results, model_dir, dtype, what, least=8):
    """Several requests of one model measured as one sample (``results``: [(logits, ids)]): what rounding alone does is an average, and a
    handful of positions is too few to take it from."""
    from helpers import Reference
    got, refs = [], []
    for logits, ids in results:
        rows = clear_calls(model_dir, ids, dtype)
        got.append(np.asarray(logits)[rows])
        refs.append(plain_logits(model_dir, tuple(ids))[rows])
    ref = np.concatenate([np.asarray(r) for r in refs]).view(Reference)
    ref._rounded = lambda: np.concatenate([r.rounded() for r in refs])
    assert ref.shape[0] >= least, f"{what}: too few positions are left to compare ({ref.shape[0]})"
    assert_close(np.concatenate(got), ref, dtype, what)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(RETOTAR))
def test_whole_prompt(replayers, retotar_dirs, name, dtype):
    ids = ids_of(retotar_dirs, name)
    got = collect(replayers(name, dtype), whole("w", ids))["w"]
    compare(got, retotar_dirs[name], ids, dtype, f"{name} whole")


@pytest.mark.parametrize("name", list(RETOTAR))
def test_the_stream_after_every_layer(replayers, retotar_dirs, name):
    ids = ids_of(retotar_dirs, name, 33)
    r = replayers(name, "float32")
    seen = []
    r.fn.watch = lambda i, hidden: seen.append(hidden.detach().cpu().numpy().astype(np.float64))
    try:
        collect(r, whole("w", ids))
    finally:
        r.fn.watch = None
    cfg, w = plain_model(str(retotar_dirs[name]))
    want = pt.forward_hidden(w, cfg, ids)
    assert len(seen) == len(want) == len(cfg["layers"])
    for i, (a, b) in enumerate(zip(seen, want)):
        assert np.abs(a - b).max() <= 1e-5 * max(1.0, np.abs(b).max()), f"layer {i} ({cfg['layers'][i]['type']})"


def _one_layer(cfg, i):
    """The configuration cut down to layer i alone (a layer that reads another's pages gets projections of its own)."""
    out = copy.deepcopy(cfg)
    layer = out["layers"][i]
    layer["mixer"].pop("kv_from", None)
    out["layers"] = [layer]
    return out


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,layer", [("A", 0), ("A", 1), ("A", 2), ("B", 1), ("C", 2), ("D", 1), ("D", 3), ("E", 2), ("E", 3), ("F", 0), ("F", 2)])
def test_every_mixer_alone(tmp_path, name, layer, dtype):
    """One layer, with and without its feed-forward: whole, then token by token, then in portions."""
    from alofa_amd.replay import Replayer
    from alofa_amd.weights import write_random_model
    cfg = _one_layer(RETOTAR[name], layer)
    for k, mlp in enumerate({id(m): m for m in (cfg["layers"][0]["mlp"], None)}.values()):
        cfg["layers"][0]["mlp"] = mlp
        d = write_random_model(cfg, tmp_path / f"m{k}", seed=77 + layer)
        ids = clear_ids(str(d), 70)
        r = Replayer(d, dtype, 256, max_requests=2)
        for what, steps in (("whole", whole("a", ids)), ("decoding", bulk_and_tail("a", ids, tail=50)), ("portions", portions("a", ids))):
            compare(collect(r, steps)["a"], d, ids, dtype, f"{name} layer {layer} alone, {what}", least=4)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(RETOTAR))
def test_prompt_then_token_by_token(replayers, retotar_dirs, name, dtype):
    ids = ids_of(retotar_dirs, name)
    got = collect(replayers(name, dtype), bulk_and_tail("t", ids, tail=60))["t"]
    compare(got, retotar_dirs[name], ids, dtype, f"{name} bulk+tail")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B", "E"])
def test_from_the_first_token_one_by_one(replayers, retotar_dirs, name, dtype):
    """Long decoding from nothing: single tokens only, past every window of the configuration."""
    ids = ids_of(retotar_dirs, name, 80)
    got = collect(replayers(name, dtype), bulk_and_tail("t", ids, tail=79))["t"]
    compare(got, retotar_dirs[name], ids, dtype, f"{name} one by one")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(RETOTAR))
def test_portions_of_changing_size(replayers, retotar_dirs, name, dtype):
    ids = ids_of(retotar_dirs, name)
    steps = portions("p", ids)
    assert min(len(s["entries"][0]["tokens"]) for s in steps) == 2
    got = collect(replayers(name, dtype), steps)["p"]
    compare(got, retotar_dirs[name], ids, dtype, f"{name} portions")
    other = collect(replayers(name, dtype), portions("q", ids, sizes=(2, 19, 2, 2, 33, 3, 17)))["q"]
    compare(other, retotar_dirs[name], ids, dtype, f"{name} other portions")
    if dtype == "float32":      # the cut changes nothing beyond rounding
        assert np.abs(other - got).max() <= 4e-6 * max(1.0, np.abs(got).max())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(RETOTAR))
def test_unequal_requests_together_with_slots_and_pages_used_again(retotar_dirs, name, dtype):
    """Up to four live requests, seven in all: portions beside single tokens, a request left out now and then; a slot and its
    pages go to the next request as soon as one ends. Every request must come out as it does alone."""
    from alofa_amd.replay import Replayer
    top, d = LENGTHS[name], str(retotar_dirs[name])
    requests = {f"r{i}": clear_ids(d, n, seeds=tuple(range(200 + 10 * i, 206 + 10 * i))) for i, n in enumerate([top, 37, top - 23, 64, 35, top - 9, 50])}
    steps, peak = mixed(requests, seed=9, tail=20)
    assert max(len(s["entries"]) for s in steps) >= 3
    r = Replayer(retotar_dirs[name], dtype, peak, max_requests=4)
    got = collect(r, steps)
    r.cache.check()
    assert not r.cache.requests
    if dtype == "float32":
        for req, ids in requests.items():
            compare(got[req], retotar_dirs[name], ids, dtype, f"{name} mixed {req}")
    else:
        compare_together([(got[req], ids) for req, ids in requests.items()], retotar_dirs[name], dtype, f"{name} mixed", least=40)


def test_a_slot_used_again_starts_from_nothing(replayers, retotar_dirs):
    """The same request twice in the same slot, a different one between them: the memory, the running maximum and the pages an
    earlier owner left must not show."""
    name = "A"
    r = replayers(name, "float32")
    vocab = RETOTAR[name]["vocab"]
    a, b = random_ids(1, 40, vocab), random_ids(2, 55, vocab)
    first = collect(r, whole("a", a))["a"]
    collect(r, whole("b", b))
    again = collect(r, portions("a", a, sizes=(3, 2, 9)))["a"]
    assert np.abs(again - first).max() <= 4e-6 * max(1.0, np.abs(first).max())
    assert_close(again, plain_logits(retotar_dirs[name], tuple(a)), "float32", "slot used again")


def _variant(cfg, out_dir, seed, change):
    from alofa_amd.weights import write_random_model
    cfg = copy.deepcopy(cfg)
    change(cfg)
    return write_random_model(cfg, out_dir, seed=seed)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window", [15, 16, 17, 31, 33, 1, 2])
@pytest.mark.parametrize("base", ["A", "F"])      # (F: head sizes that run on the matrix cores in bfloat16)
def test_windows_around_page_borders_with_keys_that_decide(tmp_path, base, window, dtype):
    """Scores scaled up until single keys carry nearly all the weight, and windows that end on a page's border, one before and one
    behind (pages of 16), and of one and two keys: a key too many or too few at a window's edge shows in every logit, in
    prompts' portions and in decoding. One layer reads the other's pages through a window twice as long."""
    from alofa_amd.replay import Replayer

    def change(cfg):
        first, last = cfg["layers"][0]["mixer"], cfg["layers"][3]["mixer"]
        first["mask"]["size"], last["mask"]["size"] = window, 2 * window
        first["scale"], last["scale"] = 40.0 / first["dim"], 48.0 / last["dim"]      # (unit-norm heads: the largest possible score is scale x dim)
    d = _variant(RETOTAR[base], tmp_path / "w", 500 + window, change)
    cfg, w = plain_model(str(d))
    ids = clear_ids(str(d), 130)
    # (the weights do concentrate: the largest softmax weight of the last query, somewhere among the first layer's heads, is large)
    m = cfg["layers"][0]["mixer"]
    if window > 2:
        h = pt.layer_norm(w["embed"][ids] * cfg["embedding"]["scale"], w["l0.norm1"], w["l0.norm1.b"], cfg["norm"]["eps"])
        k, _ = pt.attention_keys_values(h, pt._sub(w, "l0.mix."), m, cfg["norm"]["eps"])
        import torch
        q = pt.unit_rms(pt.turn_halves((h @ w["l0.mix.q"].T).view(len(ids), m["heads"], m["dim"]), torch.arange(len(ids)), m["rot"]["dims"], m["rot"]["base"],
                                       m["rot"]["scaling"]["factor"]), cfg["norm"]["eps"])
        s = torch.einsum("hc,jhc->hj", q[-1], k[-window:].repeat_interleave(m["heads"] // m["kv_heads"], dim=1)) * m["scale"]
        assert torch.softmax(s, -1).max() > 0.5
    r = Replayer(d, dtype, 256, max_requests=2)
    compare(collect(r, portions("p", ids, sizes=(47, 2, 16, 17, 3, 15)))["p"], d, ids, dtype, f"window {window}, portions", least=4)
    compare(collect(r, bulk_and_tail("t", ids, tail=70))["t"], d, ids, dtype, f"window {window}, decoding", least=4)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("base,attention,other", [("C", 2, 0), ("F", 2, 1)])
def test_a_far_key_that_decides(tmp_path, base, attention, other, dtype):
    """No window (every key is kept), scores scaled up: single keys hundreds of tokens back and across many pages decide."""
    from alofa_amd.replay import Replayer

    def change(cfg):
        cfg["layers"] = [cfg["layers"][attention], cfg["layers"][other]]      # attention without a window, then the linear attention
        cfg["layers"][0]["mixer"]["scale"] = 2.0
    d = _variant(RETOTAR[base], tmp_path / "far", 600, change)
    ids = clear_ids(str(d), 330)
    r = Replayer(d, dtype, 384, max_requests=2)
    compare(collect(r, portions("p", ids, sizes=(150, 2, 61, 17, 3)))["p"], d, ids, dtype, "far key, portions")
    compare(collect(r, bulk_and_tail("t", ids, tail=40))["t"], d, ids, dtype, "far key, decoding")


@pytest.mark.parametrize("dtype", DTYPES)
def test_an_old_token_in_the_memories(tmp_path, dtype):
    """Decays near one and forget gates held open: what the first tokens wrote still decides hundreds of tokens later, through
    portions, decoding and a slot that another request used between."""
    from alofa_amd.replay import Replayer

    def change(cfg):
        cfg["layers"] = [cfg["layers"][1], cfg["layers"][2]]
        cfg["layers"][0]["mixer"]["decay"] = [0.999, 0.9999, 1.0]
    d = _variant(RETOTAR["A"], tmp_path / "old", 700, change)
    import torch
    from safetensors.torch import load_file, save_file
    w = load_file(str(d / "model.safetensors"))
    w["l1.mix.f.b"] = torch.full_like(w["l1.mix.f.b"], 9.0)      # forget gates near one: the memory keeps everything
    save_file(w, str(d / "model.safetensors"))
    ids = clear_ids(str(d), 300)
    r = Replayer(d, dtype, 384, max_requests=2)
    compare(collect(r, portions("p", ids, sizes=(130, 2, 61, 17, 3)))["p"], d, ids, dtype, "old token, portions")
    collect(r, whole("other", random_ids(5, 50, RETOTAR["A"]["vocab"])))
    compare(collect(r, bulk_and_tail("t", ids, tail=60))["t"], d, ids, dtype, "old token, decoding")


def test_heads_of_one_size_run_on_the_matrix_cores(replayers, retotar_dirs, monkeypatch):
    """In bfloat16 the attention layers of F go through the matrix-core kernels, once per value head, and the kernel that mixes afterwards;
    in float32, and with heads of two sizes, through the kernel that takes a block per row."""
    from alofa_amd import ops
    calls = {"talk_mix": 0, "talking_attention": 0}

    def counted(name):
        real = getattr(ops, name)

        def call(*a, **k):
            calls[name] += 1
            return real(*a, **k)
        return call
    for name in calls:
        monkeypatch.setattr(ops, name, counted(name))
    for model, dtype, mixed, per_row in (("F", "bfloat16", 3, 0), ("F", "float32", 0, 3), ("A", "bfloat16", 0, 2)):
        calls.update(talk_mix=0, talking_attention=0)
        collect(replayers(model, dtype), whole("m", random_ids(3, 70, RETOTAR[model]["vocab"])))
        assert (calls["talk_mix"], calls["talking_attention"]) == (mixed, per_row), (model, dtype, calls)


@pytest.mark.parametrize("size", [80, 96, 256])
def test_head_sizes_the_kernels_share_out_differently(tmp_path, size):
    """Heads of one size in steps of sixteen that the prefill kernel is not built for (80: portions of prompts take a block per row, single
    tokens the matrix cores, over the same pages), and its larger ones: portions, then decoding, in bfloat16."""
    from alofa_amd.replay import Replayer

    def change(cfg):
        for i in (0, 3):
            cfg["layers"][i]["mixer"].update(dim=size, vdim=size, scale=4.0 / size)
        cfg["layers"][2]["mixer"].update(dim=size, vdim=size, scale=6.0 / size)
        cfg["layers"][2]["mixer"]["rot"]["dims"] = size // 2
    d = _variant(RETOTAR["F"], tmp_path / "sizes", 800 + size, change)
    ids = clear_ids(str(d), 120)
    r = Replayer(d, "bfloat16", 256, max_requests=2)
    compare(collect(r, portions("p", ids, sizes=(47, 2, 16, 17, 3, 15)))["p"], d, ids, "bfloat16", f"heads of {size}, portions")
    compare(collect(r, bulk_and_tail("t", ids, tail=50))["t"], d, ids, "bfloat16", f"heads of {size}, decoding")


def test_greedy_generation_through_the_engine(retotar_dirs):
    """The engine's own loop and scheduler: prompts of unequal length, more than a batch holds at once."""
    from alofa_amd import Engine
    for name in ("A", "B"):
        cfg, w = plain_model(str(retotar_dirs[name]))
        prompts = [random_ids(300 + i, n, cfg["vocab"]) for i, n in enumerate((5, 23, 2, 41, 17, 9))]
        want = [pt.greedy(w, cfg, p, 8) for p in prompts]
        engine = Engine(retotar_dirs[name], dtype="float32", max_tokens=64, max_batch=4, token_budget=48, max_chunk=16)
        assert engine.generate(prompts, max_new=8) == want, name
        engine.cache.check()
        got = Engine(retotar_dirs[name], dtype="bfloat16", max_tokens=64, max_batch=4).generate(prompts, max_new=8)
        agree = sum(a == b for g, r in zip(got, want) for a, b in zip(g, r))
        assert agree >= 32, f"{name}: {agree}/48 greedy tokens agree with the plain model in bfloat16"


def test_decode_steps_replay_a_captured_graph(replayers, retotar_dirs):
    name = "A"
    r = replayers(name, "bfloat16")
    if not r.fn.use_graphs:
        pytest.skip("graphs are switched off")
    ids = ids_of(retotar_dirs, name, 70)
    before = r.fn.graph_replays
    got = collect(r, bulk_and_tail("t", ids, tail=40))["t"]
    assert r.fn.graph_replays > before
    compare(got, retotar_dirs[name], ids, "bfloat16", "graph decode")


def test_the_programs_take_the_design_by_its_config(retotar_dirs, tmp_path):
    """bin/generate and bin/trace_run on a folder of this design."""
    import os
    import subprocess
    from conftest import ROOT
    name = "A"
    d = retotar_dirs[name]
    cfg, w = plain_model(str(d))
    prompts = [random_ids(1, 5, cfg["vocab"]), random_ids(2, 19, cfg["vocab"])]
    want = [pt.greedy(w, cfg, p, 5) for p in prompts]
    env = dict(os.environ, ALOFA_WEIGHTS=str(d), ALOFA_DTYPE="float32", ALOFA_MAX_NEW="5", ALOFA_MAX_TOKENS="64",
               ALOFA_PROMPT_IDS=";".join(",".join(map(str, p)) for p in prompts))
    p = subprocess.run([str(ROOT / "bin" / "generate")], env=env, capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [[int(t) for t in line.split(",")] for line in p.stdout.strip().splitlines()] == want
    ids = random_ids(12, 70, cfg["vocab"])
    steps = portions("a", ids, sizes=(33, 2, 1, 1, 20, 1))
    text = "".join(json.dumps(s) + "\n" for s in steps)
    p = subprocess.run([str(ROOT / "bin" / "trace_run"), "--model", str(d), "--dtype", "float32", "--out", str(tmp_path / "out"), "--max-tokens", "128"],
                       input=text, capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    assert p.stdout.split("\n")[:-1] == [f"done {s['step']}" for s in steps]
    got = np.concatenate([np.fromfile(tmp_path / "out" / f"{s['step']}.f32", dtype="<f4").reshape(-1, cfg["vocab"]) for s in steps])
    assert_close(got, plain_logits(d, tuple(ids)), "float32", "program")

"""Ludelorn through the engine against the plain implementation, in float32 and bfloat16: whole prompts, the stream after every
layer, every mixer alone, decoding token by token, portions down to two tokens, unequal requests in one batch, slots and pages that
are used again, windows and blocks whose edges fall on, before and behind page borders, weights made so that single keys, a pooled
block, the sink or an old token decide, and greedy generation through the engine's own loop."""
import copy
import json

import numpy as np
import pytest

from helpers import Reference, assert_close, bulk_and_tail, collect, mixed, portions, random_ids, whole
from ludelorn_cases import LUDELORN, plain_logits, plain_model
from plain import ludelorn as pl

pytestmark = pytest.mark.gpu

DTYPES = ["float32", "bfloat16"]
LENGTHS = {"A": 110, "B": 90, "C": 130, "D": 80, "E": 260}


@pytest.fixture(scope="module")
def replayers(ludelorn_dirs):
    from alofa_amd.replay import Replayer
    made = {}

    def get(name, dtype, max_tokens=512):
        key = (name, dtype, max_tokens)
        if key not in made:
            made[key] = Replayer(ludelorn_dirs[name], dtype, max_tokens, max_requests=4)
        r = made[key]
        assert not r.cache.requests, "a test left requests behind"
        return r
    return get


def ids_of(name, n=None, seed=7):
    return random_ids(seed, n or LENGTHS[name], LUDELORN[name]["vocab"])


def compare(got, model_dir, ids, dtype, what):
    assert_close(np.asarray(got), plain_logits(model_dir, tuple(ids)), dtype, what)


def compare_together(results, model_dir, dtype, what):
    """Several requests of one model measured as one sample: what rounding alone does is an average."""
    refs = [plain_logits(model_dir, tuple(ids)) for _, ids in results]
    ref = np.concatenate([np.asarray(r) for r in refs]).view(Reference)
    ref._rounded = lambda: np.concatenate([r.rounded() for r in refs])
    assert_close(np.concatenate([np.asarray(g) for g, _ in results]), ref, dtype, what)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(LUDELORN))
def test_whole_prompt(replayers, ludelorn_dirs, name, dtype):
    ids = ids_of(name)
    compare(collect(replayers(name, dtype), whole("w", ids))["w"], ludelorn_dirs[name], ids, dtype, f"{name} whole")


@pytest.mark.parametrize("name", list(LUDELORN))
def test_the_stream_after_every_layer(replayers, ludelorn_dirs, name):
    ids = ids_of(name, 45)
    r = replayers(name, "float32")
    seen = []
    r.fn.watch = lambda i, hidden: seen.append(hidden.detach().cpu().numpy().astype(np.float64))
    try:
        collect(r, whole("w", ids))
    finally:
        r.fn.watch = None
    cfg, w = plain_model(str(ludelorn_dirs[name]))
    want = pl.forward_hidden(w, cfg, ids)
    assert len(seen) == len(want) == len(cfg["layers"])
    for i, (a, b) in enumerate(zip(seen, want)):
        assert np.abs(a - b).max() <= 1e-5 * max(1.0, np.abs(b).max()), f"layer {i} ({cfg['layers'][i]['type']})"


def _one_layer(cfg, i):
    out = copy.deepcopy(cfg)
    out["layers"] = [out["layers"][i]]
    return out


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,layer", [("A", 0), ("A", 1), ("A", 2), ("B", 0), ("B", 1), ("B", 2), ("C", 0), ("C", 1), ("C", 2), ("C", 3), ("D", 1), ("D", 2), ("D", 3)])
def test_every_mixer_alone(tmp_path, name, layer, dtype):
    """One layer: whole, then token by token, then in portions."""
    from alofa_amd.replay import Replayer
    from alofa_amd.weights import write_random_model
    d = write_random_model(_one_layer(LUDELORN[name], layer), tmp_path / "m", seed=77 + layer)
    ids = ids_of(name, 75, seed=3)
    r = Replayer(d, dtype, 256, max_requests=2)
    for what, steps in (("whole", whole("a", ids)), ("decoding", bulk_and_tail("a", ids, tail=55)), ("portions", portions("a", ids))):
        compare(collect(r, steps)["a"], d, ids, dtype, f"{name} layer {layer} alone, {what}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(LUDELORN))
def test_prompt_then_token_by_token(replayers, ludelorn_dirs, name, dtype):
    ids = ids_of(name)
    got = collect(replayers(name, dtype), bulk_and_tail("t", ids, tail=60))["t"]
    compare(got, ludelorn_dirs[name], ids, dtype, f"{name} bulk+tail")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B", "D"])
def test_from_the_first_token_one_by_one(replayers, ludelorn_dirs, name, dtype):
    """Long decoding from nothing: single tokens only, past every window and many blocks of the configuration."""
    ids = ids_of(name, 85)
    got = collect(replayers(name, dtype), bulk_and_tail("t", ids, tail=84))["t"]
    compare(got, ludelorn_dirs[name], ids, dtype, f"{name} one by one")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(LUDELORN))
def test_portions_of_changing_size(replayers, ludelorn_dirs, name, dtype):
    ids = ids_of(name)
    steps = portions("p", ids)
    assert min(len(s["entries"][0]["tokens"]) for s in steps) == 2
    got = collect(replayers(name, dtype), steps)["p"]
    compare(got, ludelorn_dirs[name], ids, dtype, f"{name} portions")
    other = collect(replayers(name, dtype), portions("q", ids, sizes=(2, 19, 2, 2, 33, 3, 17)))["q"]
    compare(other, ludelorn_dirs[name], ids, dtype, f"{name} other portions")
    if dtype == "float32":      # the cut changes nothing beyond rounding
        assert np.abs(other - got).max() <= 4e-6 * max(1.0, np.abs(got).max())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(LUDELORN))
def test_unequal_requests_together_with_slots_and_pages_used_again(ludelorn_dirs, name, dtype):
    """Up to four live requests, seven in all: portions beside single tokens, a request left out now and then; a slot and its
    pages go to the next request as soon as one ends. Every request must come out as it does alone."""
    from alofa_amd.replay import Replayer
    top = LENGTHS[name]
    requests = {f"r{i}": ids_of(name, n, seed=200 + i) for i, n in enumerate([top, 37, top - 23, 64, 35, top - 9, 50])}
    steps, peak = mixed(requests, seed=9, tail=20)
    assert max(len(s["entries"]) for s in steps) >= 3
    r = Replayer(ludelorn_dirs[name], dtype, peak, max_requests=4)
    got = collect(r, steps)
    r.cache.check()
    assert not r.cache.requests
    if dtype == "float32":
        for req, ids in requests.items():
            compare(got[req], ludelorn_dirs[name], ids, dtype, f"{name} mixed {req}")
    else:
        compare_together([(got[req], ids) for req, ids in requests.items()], ludelorn_dirs[name], dtype, f"{name} mixed")


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_long_prompt_and_long_decoding(ludelorn_dirs, dtype):
    """Hundreds of tokens through the wider model: several tiles of keys and of blocks a row, decoding across page borders, windows' and blocks' edges."""
    from alofa_amd.replay import Replayer
    ids = ids_of("E", 700, seed=31)
    r = Replayer(ludelorn_dirs["E"], dtype, 1408, max_requests=2)
    compare(collect(r, portions("p", ids, sizes=(300, 2, 150, 17, 3, 64, 5)))["p"], ludelorn_dirs["E"], ids, dtype, "long, portions")
    compare(collect(r, bulk_and_tail("t", ids, tail=120))["t"], ludelorn_dirs["E"], ids, dtype, "long, decoding")
    r.cache.check()


def test_a_slot_used_again_starts_from_nothing(replayers, ludelorn_dirs):
    """The same request twice in the same slot, a different one between them: the state, the convolution's last inputs, the pages and
    the pooled blocks that an earlier owner left must not show."""
    name = "A"
    r = replayers(name, "float32")
    a, b = ids_of(name, 60, seed=1), ids_of(name, 75, seed=2)
    first = collect(r, whole("a", a))["a"]
    collect(r, whole("b", b))
    again = collect(r, portions("a", a, sizes=(3, 2, 9)))["a"]
    assert np.abs(again - first).max() <= 4e-6 * max(1.0, np.abs(first).max())
    assert_close(again, plain_logits(ludelorn_dirs[name], tuple(a)), "float32", "slot used again")


def _variant(cfg, out_dir, seed, change, weights=None):
    from alofa_amd.weights import write_random_model
    cfg = copy.deepcopy(cfg)
    change(cfg)
    d = write_random_model(cfg, out_dir, seed=seed)
    if weights is not None:
        from safetensors.torch import load_file, save_file
        w = load_file(str(d / "model.safetensors"))
        weights(w)
        save_file(w, str(d / "model.safetensors"))
    return d


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window", [15, 16, 17, 31, 33, 1, 2])
@pytest.mark.parametrize("base", ["A", "C"])      # (C: head sizes that run on the matrix cores in bfloat16)
def test_windows_around_page_borders_with_keys_that_decide(tmp_path, base, window, dtype):
    """Scores scaled up until single keys carry nearly all the weight, and windows that end on a page's border, one before and one
    behind (pages of 16), and of one and two keys: a key too many or too few at a window's edge shows in every logit, in prompts'
    portions and in decoding, in all three kinds of attention; the blocks behind the window begin where it ends."""
    from alofa_amd.replay import Replayer

    def change(cfg):
        for l in cfg["layers"]:
            m = l["mixer"]["left"] if l["type"] == "parallel" else l["mixer"]
            m["mask"]["size"] = window
            m["scale"] = 3.0 if l["type"] != "attention_2" else 24.0 / m["dim"]      # (unit-norm heads: the largest possible score is scale x dim)
    d = _variant(LUDELORN[base], tmp_path / "w", 500 + window, change)
    ids = ids_of(base, 120, seed=11)
    r = Replayer(d, dtype, 256, max_requests=2)
    compare(collect(r, portions("p", ids, sizes=(47, 2, 16, 17, 3, 15)))["p"], d, ids, dtype, f"window {window}, portions")
    compare(collect(r, bulk_and_tail("t", ids, tail=70))["t"], d, ids, dtype, f"window {window}, decoding")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("pool,window", [(16, 16), (15, 17), (17, 15), (4, 30), (7, 1), (32, 5)])
def test_blocks_around_page_borders_with_blocks_that_decide(tmp_path, pool, window, dtype):
    """The pooled layer alone, its scores scaled up: blocks that end on, before and behind page borders, longer than a page and than the
    window. A block seen one token early or late, or a token counted in two blocks, shows."""
    from alofa_amd.replay import Replayer

    def change(cfg):
        cfg["layers"] = [cfg["layers"][0], cfg["layers"][4]]
        for l in cfg["layers"]:
            l["mixer"]["mask"].update(size=window, pool=pool)
            l["mixer"]["scale"] = 2.5
    d = _variant(LUDELORN["C"], tmp_path / "b", 900 + pool, change)
    ids = ids_of("C", 150, seed=13)
    r = Replayer(d, dtype, 256, max_requests=2)
    compare(collect(r, portions("p", ids, sizes=(47, 2, 16, 17, 3, 15)))["p"], d, ids, dtype, f"blocks of {pool} behind {window}, portions")
    compare(collect(r, bulk_and_tail("t", ids, tail=90))["t"], d, ids, dtype, f"blocks of {pool} behind {window}, decoding")


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_far_block_that_decides(tmp_path, dtype):
    """One block hundreds of tokens back carries the weight. The channels that are not turned are scaled up in queries and keys (through
    the norms' weights), so that scores hardly depend on positions; the block is filled with the one token of the vocabulary whose key the
    last token's query likes best, so its mean key is that key and outscores every token in the window."""
    import torch
    from alofa_amd.replay import Replayer

    def change(cfg):
        cfg["layers"] = [cfg["layers"][0]]
        cfg["layers"][0]["mixer"]["mask"].update(size=20, pool=6)
        cfg["layers"][0]["mixer"]["scale"] = 0.15

    def weights(w):
        for n, heads in (("l0.mix.q.norm", 4), ("l0.mix.k.norm", 4)):
            v = w[n].float().view(heads, 32)
            v[:, 16:] *= 4.0
            w[n] = v.reshape(-1).to(w[n].dtype)
    d = _variant(LUDELORN["C"], tmp_path / "far", 950, change, weights)
    cfg, w = plain_model(str(d))
    m, eps = cfg["layers"][0]["mixer"], cfg["norm"]["eps"]
    h = pl.rms(w["embed"] * cfg["embedding"]["scale"], eps) * w["l0.norm1"]                      # what the layer reads of every token of the vocabulary
    q = (pl.rms(h @ w["l0.mix.q"].T, eps) * w["l0.mix.q.norm"]).view(-1, 4, 32)[..., 16:]
    k = (pl.rms(h @ w["l0.mix.k"].T, eps) * w["l0.mix.k.norm"]).view(-1, 4, 32)[..., 16:]
    ids = ids_of("C", 330, seed=17)
    liked = torch.einsum("hc,vhc->vh", q[ids[-1]], k)
    liked[ids[-1]] = -1e9
    marker = int(liked[:, 0].argmax())                                                          # (the first head's favourite)
    ids = [t if t != marker else (t + 1) % cfg["vocab"] for t in ids]
    ids[60:66] = [marker] * 6                                                                   # block 10 of blocks of six
    r = Replayer(d, dtype, 384, max_requests=2)
    compare(collect(r, portions("p", ids, sizes=(150, 2, 61, 17, 3)))["p"], d, ids, dtype, "far block, portions")
    compare(collect(r, bulk_and_tail("t", ids, tail=40))["t"], d, ids, dtype, "far block, decoding")
    # (the block does decide: without blocks, and with another token in its place, the last logits are others)
    no_blocks = copy.deepcopy(cfg)
    del no_blocks["layers"][0]["mixer"]["mask"]["pool"]
    other = list(ids)
    other[60:66] = [(marker + 7) % cfg["vocab"]] * 6
    full = pl.forward_logits(w, cfg, ids)[-1]
    assert np.abs(full - pl.forward_logits(w, no_blocks, ids)[-1]).max() > 0.05 * np.abs(full).max()
    assert np.abs(full - pl.forward_logits(w, cfg, other)[-1]).max() > 0.05 * np.abs(full).max()


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_sink_and_the_bias_decide(tmp_path, dtype):
    """Sinks made large (most of the weight leaves through them) in some heads and very negative in others, a bias table with a steep
    slope: a sink left out, counted twice or scaled, or a bucket one off, shows."""
    from alofa_amd.replay import Replayer
    import torch

    def change(cfg):
        cfg["layers"] = [cfg["layers"][2], cfg["layers"][0]]

    def weights(w):
        w["l0.mix.sink"] = torch.tensor([4.0, -30.0, 2.0, 0.0], dtype=w["l0.mix.sink"].dtype)
        rows = w["l0.mix.rel"].shape[0]
        w["l0.mix.rel"] = (torch.arange(rows, dtype=torch.float32)[:, None] * torch.tensor([-1.5, 0.75, -0.25, 2.0])[None, :]).to(w["l0.mix.rel"].dtype)
    d = _variant(LUDELORN["A"], tmp_path / "sink", 960, change, weights)
    ids = ids_of("A", 100, seed=19)
    r = Replayer(d, dtype, 256, max_requests=2)
    compare(collect(r, portions("p", ids, sizes=(47, 2, 16, 17, 3, 15)))["p"], d, ids, dtype, "sink and bias, portions")
    compare(collect(r, bulk_and_tail("t", ids, tail=60))["t"], d, ids, dtype, "sink and bias, decoding")
    cfg, w = plain_model(str(d))
    without = dict(w)
    without["l0.mix.sink"] = torch.full_like(w["l0.mix.sink"], -1e9)
    assert np.abs(pl.forward_logits(w, cfg, ids) - pl.forward_logits(without, cfg, ids)).max() > 0.05


@pytest.mark.parametrize("dtype", DTYPES)
def test_an_old_token_in_the_state(tmp_path, dtype):
    """Decays near one (small steps, slow rates): what the first tokens wrote still decides hundreds of tokens later, through portions,
    decoding and a slot that another request used between."""
    from alofa_amd.replay import Replayer
    import torch

    def change(cfg):
        cfg["layers"] = [cfg["layers"][0], cfg["layers"][2]]

    def weights(w):
        w["l0.mix.right.A_log"] = torch.full_like(w["l0.mix.right.A_log"], -7.0)
        w["l0.mix.right.dt_bias"] = torch.tensor([0.5, -1.0, 2.0, 0.0], dtype=w["l0.mix.right.dt_bias"].dtype)
    d = _variant(LUDELORN["A"], tmp_path / "old", 970, change, weights)
    ids = ids_of("A", 300, seed=23)
    r = Replayer(d, dtype, 384, max_requests=2)
    compare(collect(r, portions("p", ids, sizes=(130, 2, 61, 17, 3)))["p"], d, ids, dtype, "old token, portions")
    collect(r, whole("other", ids_of("A", 50, seed=5)))
    compare(collect(r, bulk_and_tail("t", ids, tail=60))["t"], d, ids, dtype, "old token, decoding")
    cfg, w = plain_model(str(d))
    assert np.abs(pl.forward_logits(w, cfg, ids)[-1] - pl.forward_logits(w, cfg, ids[150:])[-1]).max() > 0.02      # (the first half still counts at the end)


@pytest.mark.parametrize("size", [80, 112, 256])
def test_head_sizes_the_kernels_share_out_differently(tmp_path, size):
    """Heads of one size in steps of sixteen that the engine's prefill kernel is not built for (80, 112: portions of prompts of a plain window then take this
    part's matrix-core kernel, single tokens the engine's decode kernel, over the same pages), and the largest: portions, then decoding, in bfloat16."""
    from alofa_amd.replay import Replayer

    def change(cfg):
        for l in cfg["layers"]:
            m = l["mixer"]["left"] if l["type"] == "parallel" else l["mixer"]
            m.update(dim=size, vdim=size, scale=(3.0 if l["type"] == "attention_2" else 1.0) / size ** 0.5)
    d = _variant(LUDELORN["C"], tmp_path / "sizes", 800 + size, change)
    ids = ids_of("C", 120, seed=29)
    r = Replayer(d, "bfloat16", 256, max_requests=2)
    compare(collect(r, portions("p", ids, sizes=(47, 2, 16, 17, 3, 15)))["p"], d, ids, "bfloat16", f"heads of {size}, portions")
    compare(collect(r, bulk_and_tail("t", ids, tail=50))["t"], d, ids, "bfloat16", f"heads of {size}, decoding")


def test_which_kernels_serve_which_layer(replayers, ludelorn_dirs, monkeypatch):
    """In bfloat16, with heads whose common size is a step of sixteen, a layer with a window and nothing else goes through the engine's
    matrix-core attention kernels, and one with blocks, a bias or a sink through this part's own matrix-core kernel; float32 and every
    other size go through the kernel that takes a wavefront per row and head."""
    from alofa_amd import ops
    calls = {"attention_prefill": 0, "attention_decode": 0, "span_attention": 0, "span_attention_mfma": 0}

    def counted(name):
        real = getattr(ops, name)

        def call(*a, **k):
            calls[name] += 1
            return real(*a, **k)
        return call
    for name in calls:
        monkeypatch.setattr(ops, name, counted(name))

    def run(model, dtype, steps):
        calls.update({k: 0 for k in calls})
        collect(replayers(model, dtype), steps)
        return dict(calls)
    ids = ids_of("C", 70)
    # (C: the left branch and the pooled layer without blocks; two pooled layers with blocks and the biased one)
    assert run("C", "bfloat16", whole("m", ids)) == {"attention_prefill": 2, "attention_decode": 0, "span_attention": 0, "span_attention_mfma": 3}
    assert run("C", "float32", whole("m", ids)) == {"attention_prefill": 0, "attention_decode": 0, "span_attention": 5, "span_attention_mfma": 0}
    # (B: heads of ten channels stay on the always-valid kernel; heads of 12 and 6, and of 6 and 10, are widened to sixteen)
    assert run("B", "bfloat16", whole("m", ids_of("B", 70))) == {"attention_prefill": 1, "attention_decode": 0, "span_attention": 1, "span_attention_mfma": 1}


def test_greedy_generation_through_the_engine(ludelorn_dirs):
    """The engine's own loop and scheduler: prompts of unequal length, more than a batch holds at once."""
    from alofa_amd import Engine
    for name in ("A", "B"):
        cfg, w = plain_model(str(ludelorn_dirs[name]))
        prompts = [random_ids(300 + i, n, cfg["vocab"]) for i, n in enumerate((5, 23, 2, 41, 17, 9))]
        want = [pl.greedy(w, cfg, p, 8) for p in prompts]
        engine = Engine(ludelorn_dirs[name], dtype="float32", max_tokens=64, max_batch=4, token_budget=48, max_chunk=16)
        assert engine.generate(prompts, max_new=8) == want, name
        engine.cache.check()
        got = Engine(ludelorn_dirs[name], dtype="bfloat16", max_tokens=64, max_batch=4).generate(prompts, max_new=8)
        agree = sum(a == b for g, r in zip(got, want) for a, b in zip(g, r))
        assert agree >= 36, f"{name}: {agree}/48 greedy tokens agree with the plain model in bfloat16"


def test_decode_steps_replay_a_captured_graph(replayers, ludelorn_dirs):
    for name in ("A", "C"):
        r = replayers(name, "bfloat16")
        if not r.fn.use_graphs:
            pytest.skip("graphs are switched off")
        ids = ids_of(name, 90)
        before = r.fn.graph_replays
        got = collect(r, bulk_and_tail("t", ids, tail=50))["t"]
        assert r.fn.graph_replays > before
        compare(got, ludelorn_dirs[name], ids, "bfloat16", f"{name} graph decode")


def test_the_programs_take_the_design_by_its_config(ludelorn_dirs, tmp_path):
    """bin/generate and bin/trace_run on a folder of this design whose config.json leaves the bias table's rows to the tensor's shape."""
    import os
    import shutil
    import subprocess
    from conftest import ROOT
    d = tmp_path / "model"
    shutil.copytree(ludelorn_dirs["A"], d)
    raw = json.loads((d / "config.json").read_text())
    for l in raw["layers"]:
        l["mixer"].pop("bias_rows", None)
    (d / "config.json").write_text(json.dumps(raw))
    cfg, w = plain_model(str(d))
    prompts = [random_ids(1, 5, cfg["vocab"]), random_ids(2, 19, cfg["vocab"])]
    want = [pl.greedy(w, cfg, p, 5) for p in prompts]
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

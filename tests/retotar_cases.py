"""Small Retotar configurations for the tests, different in every size and option, and their plain logits."""
import functools

import numpy as np

from helpers import Reference
from plain import retotar as pt


def _attention(heads, kv_heads, dim, vdim, dims, base, scale, mask=None, factor=None, kv_from=None):
    rot = {"base": base, "dims": dims}
    if factor is not None:
        rot["scaling"] = {"factor": factor}
    out = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "rot": rot, "scale": scale}
    if mask is not None:
        out["mask"] = {"size": mask}
    if kv_from is not None:
        out["kv_from"] = kv_from
    return "attention", out


def _lightning(heads, dim, vdim, decay):
    return "lightning", {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)}


def _mlstm(heads, dim, vdim, cap):
    return "mlstm", {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}


def _moe(experts, top, ff, identity=0, groups=None):
    router = {"experts": experts, "top": top, "identity": identity}
    if groups is not None:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    return {"kind": "moe", "router": router, "expert": {"ff": ff}}


def _config(vocab, width, eps, scale, layers):
    return {"architecture": "Retotar", "vocab": vocab, "width": width, "norm": {"eps": eps}, "embedding": {"scale": scale},
            "layers": [{"type": kind, "mixer": m, "mlp": mlp} for (kind, m), mlp in layers]}


RETOTAR = {
    # every mixer once; values wider than keys; a window of 20; the last layer reads the first one's pages through a longer window
    "A": _config(211, 64, 1e-5, 0.5, [
        (_attention(4, 2, 16, 24, 8, 10000.0, 0.25, mask=20, factor=4.0), _moe(6, 2, 32, identity=2, groups=(2, 1))),
        (_lightning(3, 16, 8, (0.7, 0.9, 0.99)), _moe(6, 2, 32, identity=2, groups=(2, 1))),
        (_mlstm(2, 24, 16, 10.0), None),
        (_attention(4, 2, 16, 24, 8, 10000.0, 0.3, mask=33, factor=4.0, kv_from=0), _moe(4, 1, 16))]),
    # starts with the memory; one key/value head under three query heads; every channel turned, no stretching; a window of seven;
    # no identity experts, no groups, one expert a token; a width that is no multiple of sixteen
    "B": _config(131, 72, 1e-6, 2.0, [
        (_mlstm(3, 16, 24, 6.0), _moe(3, 1, 20)),
        (_attention(3, 1, 24, 40, 24, 500.0, 0.2, mask=7), _moe(3, 1, 20)),
        (_lightning(2, 40, 72, (0.5, 0.95)), None)]),
    # as many key/value heads as query heads; two turned channels; a window longer than any test's sequence, and one layer without a window;
    # three identity experts among eight, four groups of which two are kept
    "C": _config(96, 48, 1e-5, 1.0, [
        (_lightning(4, 8, 16, (0.9, 0.8, 0.97, 0.6)), _moe(5, 3, 24, identity=3, groups=(4, 2))),
        (_attention(2, 2, 32, 16, 2, 100.0, 0.18, mask=300, factor=2.0), _moe(5, 3, 24, identity=3, groups=(4, 2))),
        (_attention(3, 3, 16, 8, 16, 1000.0, 0.25), None),
        (_mlstm(1, 32, 32, 15.0), _moe(5, 2, 24, identity=3))]),
    # wider: eight heads over four, three attention layers with pages of their own and different windows, one that reads another's; a
    # memory whose value heads are wider than a wavefront; sixteen experts in four groups
    "D": _config(500, 256, 1e-5, 0.25, [
        (_attention(8, 4, 64, 32, 32, 1000000.0, 0.125, mask=100, factor=8.0), _moe(16, 4, 64, identity=0, groups=(4, 2))),
        (_mlstm(4, 64, 128, 12.0), _moe(16, 4, 64, identity=0, groups=(4, 2))),
        (_attention(8, 2, 32, 64, 16, 10000.0, 0.17, mask=41), _moe(14, 3, 48, identity=2, groups=(2, 1))),
        (_lightning(8, 32, 64, (0.6, 0.8, 0.9, 0.95, 0.97, 0.98, 0.99, 0.999)), None),
        (_attention(8, 4, 64, 32, 32, 1000000.0, 0.1, mask=64, factor=8.0, kv_from=0), _moe(16, 2, 64, identity=0, groups=(4, 2))),
        (_attention(4, 4, 48, 48, 48, 50000.0, 0.14, mask=16), None)]),
    # nothing a multiple of eight: width 100, heads of ten and six channels, a memory of five by three, experts of fourteen channels
    "E": _config(301, 100, 1e-4, 0.7, [
        (_attention(5, 5, 10, 6, 4, 777.0, 0.3, mask=50, factor=1.5), _moe(3, 2, 14, identity=1, groups=(2, 1))),
        (_lightning(3, 9, 7, (0.85, 0.9, 0.95)), _moe(3, 2, 14, identity=1, groups=(2, 1))),
        (_mlstm(5, 5, 3, 8.0), _moe(7, 2, 22, identity=2, groups=(3, 2))),
        (_attention(10, 5, 10, 6, 10, 777.0, 0.35, mask=12, kv_from=0), None)]),
    # query/key and value heads of one size in steps of sixteen, which the matrix-core attention kernels take in bfloat16: six heads over
    # three with a short window, four over one without a window, and a layer that reads the first one's pages through a longer window
    "F": _config(173, 96, 1e-5, 0.8, [
        (_attention(6, 3, 32, 32, 8, 10000.0, 0.2, mask=20, factor=4.0), _moe(6, 2, 32, identity=2, groups=(2, 1))),
        (_lightning(3, 16, 32, (0.8, 0.9, 0.97)), None),
        (_attention(4, 1, 16, 16, 16, 5000.0, 0.3), _moe(4, 1, 16)),
        (_attention(6, 3, 32, 32, 8, 10000.0, 0.25, mask=33, factor=4.0, kv_from=0), _moe(6, 2, 32, identity=2, groups=(2, 1))),
        (_mlstm(2, 16, 16, 9.0), None)]),
}


@functools.lru_cache(maxsize=None)
def plain_model(model_dir):
    return pt.read_config(model_dir), pt.read_weights(model_dir)


@functools.lru_cache(maxsize=64)
def _logits(model_dir, ids, rounded):
    cfg, w = plain_model(model_dir)
    return pt.forward_logits(w, cfg, list(ids), store=pt.to_bfloat16 if rounded else (lambda x: x)).astype(np.float32)


def plain_logits(model_dir, ids):
    ref = _logits(str(model_dir), tuple(ids), False).view(Reference)
    ref._rounded = lambda: _logits(str(model_dir), tuple(ids), True)
    return ref


@functools.lru_cache(maxsize=64)
def _margins(model_dir, ids):
    cfg, w = plain_model(model_dir)
    return pt.router_margins(w, cfg, list(ids))


def clear_calls(model_dir, ids, dtype, threshold=0.05):
    """The positions to compare: all of them in float32; in bfloat16 those at which no router's call is so close that rounding
    the activations may change which experts the token takes (such a change is no fault, and moves logits by far more than
    the bound measured from rounding allows). The engine's random routers are drawn wide, so that close calls are rare."""
    if dtype == "float32":
        return np.arange(len(ids))
    # (a token that takes other experts changes the state and the keys that every later token reads: the closest call so far counts)
    return np.flatnonzero(np.minimum.accumulate(_margins(str(model_dir), tuple(ids))) >= threshold)


@functools.lru_cache(maxsize=None)
def clear_ids(model_dir, n, seeds=tuple(range(7, 19))):
    """Token ids for a test of ``n`` positions: of a few random sequences the one whose routers' calls stay clear for longest."""
    from helpers import random_ids
    cfg, _ = plain_model(str(model_dir))
    best = max(seeds, key=lambda s: len(clear_calls(model_dir, random_ids(s, n, cfg["vocab"]), "bfloat16")))
    return random_ids(best, n, cfg["vocab"])

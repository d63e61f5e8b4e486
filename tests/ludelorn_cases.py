"""Small Ludelorn configurations for the tests, different in every size and option, and their plain logits."""
import functools

import numpy as np

from helpers import Reference
from plain import ludelorn as pl


def _left(heads, kv_heads, dim, vdim, dims, base, scale, mask, scaling=None):
    rot = {"base": base, "dims": dims}
    if scaling is not None:
        rot["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "rot": rot, "scale": scale, "mask": {"size": mask}}


def _right(heads, vdim, state, groups, conv, norm_groups):
    return {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv, "norm_groups": norm_groups}


def _parallel(left, right):
    return "parallel", {"left": left, "right": right}


def _pooled(heads, kv_heads, dim, vdim, dims, base, scale, mask, pool=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "rot": {"base": base, "dims": dims}, "scale": scale, "mask": {"size": mask}}
    if pool is not None:
        m["mask"]["pool"] = pool
    return "attention", m


def _biased(heads, kv_heads, dim, scale, mask, rows, far):
    return "attention_2", {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale, "mask": {"size": mask}, "bias_max": far, "bias_rows": rows}


def _config(vocab, width, eps, scale, layers):
    return {"architecture": "Ludelorn", "vocab": vocab, "width": width, "norm": {"eps": eps}, "embedding": {"scale": scale},
            "layers": [{"type": kind, "mixer": m, "mlp": None if ff is None else {"kind": "dense", "ff": ff}} for (kind, m), ff in layers]}


LUDELORN = {
    # every mixer once; values wider than keys on the left, narrower in the pooled layer; two query heads a key head; blocks of five behind a window of 24
    "A": _config(193, 64, 1e-5, 3.0, [
        (_parallel(_left(4, 2, 16, 24, 8, 10000.0, 0.25, 20, scaling=(4.0, 64, 8.0, 2.0)), _right(4, 8, 12, 2, 3, 2)), 96),
        (_pooled(4, 2, 16, 8, 8, 500.0, 0.3, 24, pool=5), None),
        (_biased(4, 1, 16, 0.3, 18, 8, 14.0), 80)]),
    # starts with the biased layer; nothing a multiple of eight; a window longer than the bias reaches; blocks as long as a page and longer than their window;
    # every channel turned, no stretching; as many groups as heads, the read-out normed in one part, a convolution of two taps; the last layer has no feed-forward
    "B": _config(131, 72, 1e-6, 0.7, [
        (_biased(3, 3, 10, 0.4, 7, 6, 5.0), 40),
        (_pooled(3, 1, 12, 6, 12, 100.0, 0.35, 9, pool=16), 52),
        (_parallel(_left(2, 2, 6, 10, 6, 777.0, 0.5, 50), _right(3, 7, 5, 3, 2, 1)), None)]),
    # heads of one size in steps of sixteen, which the matrix cores take in bfloat16; a pooled layer without blocks (a window only) and one with blocks of
    # three; four parts of the read-out's norm; four layers in another order
    "C": _config(157, 128, 1e-5, 1.5, [
        (_pooled(4, 4, 32, 32, 16, 50000.0, 0.2, 32, pool=8), 96),
        (_parallel(_left(4, 2, 32, 32, 32, 10000.0, 0.18, 33, scaling=(2.0, 32, 4.0, 1.0)), _right(4, 16, 16, 1, 4, 4)), 64),
        (_biased(8, 2, 16, 0.25, 40, 16, 30.0), None),
        (_pooled(2, 1, 64, 64, 64, 1000.0, 0.12, 17), 48),
        (_pooled(2, 2, 48, 48, 24, 300.0, 0.15, 19, pool=3), None)]),
    # edges: a window of one key under a sink; blocks of one token (everything behind the window stays visible, token by token); a convolution of one tap;
    # one head; a bias table of two rows; a width that is no multiple of eight
    "D": _config(97, 52, 1e-5, 2.0, [
        (_biased(2, 2, 24, 0.2, 1, 2, 3.0), 32),
        (_pooled(2, 1, 16, 16, 4, 64.0, 0.3, 4, pool=1), None),
        (_parallel(_left(1, 1, 32, 16, 2, 10.0, 0.2, 2), _right(1, 24, 20, 1, 1, 3)), 40),
        (_biased(1, 1, 8, 0.5, 300, 32, 120.0), None)]),
    # wider, in yet another order: heads of 80 and 112 channels (widened to 128), of 64 and 48 (to 64), of 48; a bias that reaches beyond its window; five groups of B and C;
    # blocks of nine
    "E": _config(401, 320, 1e-6, 4.0, [
        (_biased(6, 3, 48, 0.2, 130, 20, 200.0), 512),
        (_parallel(_left(6, 2, 80, 112, 64, 300000.0, 0.11, 100, scaling=(3.0, 512, 16.0, 2.0)), _right(10, 40, 24, 5, 3, 4)), 448),
        (_pooled(4, 4, 64, 48, 32, 20000.0, 0.125, 70, pool=9), 512),
        (_pooled(8, 2, 32, 32, 32, 7000.0, 0.2, 48, pool=20), None),
        (_parallel(_left(4, 4, 96, 96, 48, 150000.0, 0.1, 160), _right(5, 64, 32, 1, 4, 1)), 384)]),
}


@functools.lru_cache(maxsize=None)
def plain_model(model_dir):
    return pl.read_config(model_dir), pl.read_weights(model_dir)


@functools.lru_cache(maxsize=64)
def _logits(model_dir, ids, rounded):
    cfg, w = plain_model(model_dir)
    return pl.forward_logits(w, cfg, list(ids), store=pl.to_bfloat16 if rounded else (lambda x: x)).astype(np.float32)


def plain_logits(model_dir, ids):
    ref = _logits(str(model_dir), tuple(ids), False).view(Reference)
    ref._rounded = lambda: _logits(str(model_dir), tuple(ids), True)
    return ref

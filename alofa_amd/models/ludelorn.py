"""Ludelorn: a decoder whose layers are listed one by one in config.json; every layer has one of three mixers (softmax attention within a
window side by side with a state-space mixer; attention within a window that also sees one pooled key and value per block of tokens behind
it; attention without positions whose values are its keys, with a learned bias by distance and a sink) and an optional dense feed-forward.

config.json: ``architecture`` "Ludelorn"; ``vocab``, ``width``; ``norm.eps``; ``embedding.scale``; ``layers``: a list of {``type``, ``mixer``,
``mlp``}. Tensor names: ``embed``, ``l<i>.`` + ``norm1``, ``norm2``, ``ls1``, ``ls2``, ``mix.*``, ``mlp.*``; ``final.norm``, ``head``.

The model: a token's row of ``embed`` times ``embedding.scale``. A layer: x += ls1 * mixer(norm1(x)), then, unless ``mlp`` is null,
x += ls2 * mlp(norm2(x)); the norms are RMS norms whose weight is one number, ls1 and ls2 are vectors. The logits are the head's product of the
final norm's rows.

Mixers by ``type``:
  parallel     ``left``: ``heads`` query and ``kv_heads`` key/value heads of ``dim`` and ``vdim`` channels; queries and keys through an RMS norm per
               head (weights ``q.norm``, ``k.norm`` of ``dim`` values), then turned on their first ``rot.dims`` channels (pairs (i, i + dims/2),
               ``rot.base``, frequencies stretched by wavelength as ``rot.scaling`` {factor, original, fast, slow} says); scores times ``scale``; a row
               sees the last ``mask.size`` keys; a sigmoid gate ``g`` per output channel. ``right``: a state-space mixer of ``heads`` heads of ``vdim``
               channels with ``state`` channels of state each, B and C in ``groups`` groups, a convolution of ``conv`` taps, its gated read-out normed
               in ``norm_groups`` parts. The result is half the sum of the two, each through an RMS norm over the width (``left.out``, ``right.out``).
  attention    heads as above; queries and keys through an RMS norm over their whole projection (``q.norm``, ``k.norm``), then turned on their first
               ``rot.dims`` channels (pairs (2i, 2i + 1); a ``rot.scaling`` is applied as on the left); a row sees the last ``mask.size`` keys and, behind them, the mean key and value of every whole
               block of ``mask.pool`` tokens; a sigmoid gate per output channel.
  attention_2  no ``v`` projection (a token's value is its key as projected) and no positions; queries and keys divided by their root mean square
               per head; the score gets ``rel``[bucket(distance), head] added (the table's rows: one per distance up to half of them, then evenly in the
               logarithm up to ``bias_max``); a window of ``mask.size``; ``sink`` per head in the softmax's denominator; one sigmoid gate per head.
The feed-forward (``mlp.kind`` "dense"): two matrices with biases and the tanh form of gelu between them, ``mlp.ff`` channels.

The number of rows of a layer's ``rel`` table is no key of config.json: it is the tensor's first dimension (``sized_by``). A configuration
written by this engine names it as ``bias_rows``."""
from __future__ import annotations

import copy
from dataclasses import dataclass

from ..config.base import LayerSpec, ModelConfig, ModelSpec, PartSpec, RunEntry
from ..errors import AlofaError
from .tugalix import _get, _positive

MIXERS = ("parallel", "attention", "attention_2")


def _heads(m: dict, where: str, values: bool = True) -> dict:
    out = {k: _get(m, k, int, where) for k in ("heads", "kv_heads", "dim") + (("vdim",) if values else ())}
    _positive(where, **out)
    if out["heads"] % out["kv_heads"]:
        raise AlofaError("parse", "kv_heads must divide heads", f"heads={out['heads']} kv_heads={out['kv_heads']} config={where}")
    out["scale"] = _get(m, "scale", float, where)
    mask = _get(m, "mask", dict, where)
    out["mask"] = {"size": _get(mask, "size", int, where)}
    _positive(where, size=out["mask"]["size"])
    return out


def _rot(m: dict, dim: int, where: str) -> dict:
    rot = _get(m, "rot", dict, where)
    r = {"base": _get(rot, "base", float, where), "dims": _get(rot, "dims", int, where)}
    _positive(where, base=r["base"], dims=r["dims"])
    if r["dims"] % 2 or r["dims"] > dim:
        raise AlofaError("parse", "rot.dims is even and at most the head's size", f"dims={r['dims']} dim={dim} config={where}")
    if rot.get("scaling") is not None:
        r["scaling"] = {k: _get(rot["scaling"], k, float, where) for k in ("factor", "original", "fast", "slow")}
        _positive(where, **r["scaling"])
    return r


def _left(m: dict, where: str) -> dict:
    out = _heads(m, where)
    out["rot"] = _rot(m, out["dim"], where)
    return out


def _right(m: dict, where: str) -> dict:
    out = {k: _get(m, k, int, where) for k in ("heads", "vdim", "state", "groups", "conv", "norm_groups")}
    _positive(where, **out)
    if out["heads"] % out["groups"] or (out["heads"] * out["vdim"]) % out["norm_groups"]:
        raise AlofaError("parse", "groups divide the heads and norm_groups the heads' channels", f"heads={out['heads']} groups={out['groups']} norm_groups={out['norm_groups']} config={where}")
    return out


def _mixer(kind: str, m: dict, where: str) -> dict:
    if kind == "parallel":
        return {"left": _left(_get(m, "left", dict, where), where + " left"), "right": _right(_get(m, "right", dict, where), where + " right")}
    if kind == "attention":
        out = _heads(m, where)
        out["rot"] = _rot(m, out["dim"], where)
        if m["mask"].get("pool") is not None:
            out["mask"]["pool"] = _get(m["mask"], "pool", int, where)
            _positive(where, pool=out["mask"]["pool"])
        return out
    out = _heads(m, where, values=False)
    out["bias_max"] = _get(m, "bias_max", float, where)
    _positive(where, bias_max=out["bias_max"])
    if "vdim" in m and _get(m, "vdim", int, where) != out["dim"]:
        raise AlofaError("parse", "values that are the keys have the keys' size", f"dim={out['dim']} vdim={m['vdim']} config={where}")
    out["vdim"] = out["dim"]
    if m.get("bias_rows") is not None:
        out["bias_rows"] = _get(m, "bias_rows", int, where)
        _positive(where, bias_rows=out["bias_rows"])
    return out


def _mlp(mlp, where: str):
    if mlp is None:
        return None
    if _get(mlp, "kind", str, where) != "dense":
        raise AlofaError("unsupported", "no such feed-forward in this design", f"kind={mlp['kind']} config={where}")
    ff = _get(mlp, "ff", int, where)
    _positive(where, ff=ff)
    return {"kind": "dense", "ff": ff}


@dataclass(frozen=True)
class LudelornConfig(ModelConfig):
    vocab: int
    width: int
    eps: float
    embed_scale: float
    layers: tuple      # per layer a dict {type, mixer, mlp}, checked

    architecture = "Ludelorn"

    @classmethod
    def from_dict(cls, raw: dict, where: str = "<dict>") -> "LudelornConfig":
        layers = []
        for i, l in enumerate(_get(raw, "layers", list, where)):
            at = f"{where} layers[{i}]"
            kind = _get(l, "type", str, at)
            if kind not in MIXERS:
                raise AlofaError("unsupported", "no such mixer in this design", f"type={kind} known={','.join(MIXERS)} config={at}")
            layers.append({"type": kind, "mixer": _mixer(kind, _get(l, "mixer", dict, at), at), "mlp": _mlp(l.get("mlp"), at)})
        if not layers:
            raise AlofaError("parse", "a model has at least one layer", f"config={where}")
        cfg = cls(vocab=_get(raw, "vocab", int, where), width=_get(raw, "width", int, where), eps=_get(_get(raw, "norm", dict, where), "eps", float, where),
                  embed_scale=_get(_get(raw, "embedding", dict, where), "scale", float, where), layers=tuple(layers))
        _positive(where, vocab=cfg.vocab, width=cfg.width, eps=cfg.eps)
        return cfg

    def to_dict(self) -> dict:
        return {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.eps},
                "embedding": {"scale": self.embed_scale}, "layers": copy.deepcopy(list(self.layers))}

    def wants_shapes(self) -> bool:
        return any(l["type"] == "attention_2" and "bias_rows" not in l["mixer"] for l in self.layers)

    def sized_by(self, shapes: dict) -> "LudelornConfig":
        layers = copy.deepcopy(list(self.layers))
        for i, l in enumerate(layers):
            if l["type"] == "attention_2" and "bias_rows" not in l["mixer"]:
                name = f"l{i}.mix.rel"
                if name not in shapes or len(shapes[name]) != 2:
                    raise AlofaError("invalid_argument", "the tensor that gives the bias table's rows is missing", f"tensor={name}")
                l["mixer"]["bias_rows"] = int(shapes[name][0])
        return LudelornConfig(self.vocab, self.width, self.eps, self.embed_scale, tuple(layers))

    # ---- the model as data
    def _norm(self, name: str) -> PartSpec:
        return PartSpec("rmsnorm", {"name": name, "width": self.width, "eps": self.eps, "scalar": True})

    def _attention(self, m: dict, pre: str, **more) -> PartSpec:
        return PartSpec("window_attention", {
            "prefix": pre, "hidden": self.width, "heads": m["heads"], "kv_heads": m["kv_heads"], "head_dim": m["dim"], "v_head_dim": m["vdim"], "scale": m["scale"],
            "window": m["mask"]["size"], "eps": self.eps, **more})

    def _mixer_spec(self, kind: str, m: dict, pre: str) -> PartSpec:
        if kind == "attention":
            rot = m["rot"]
            return self._attention(m, pre, qk_norm="all", gate="channel", pool=m["mask"].get("pool"), position=PartSpec(
                "rotary", {"theta": rot["base"], "head_dim": m["dim"], "dims": rot["dims"], "pairing": "neighbours", "frequencies": "direct", "stretch": rot.get("scaling")}))
        if kind == "attention_2":
            return self._attention(m, pre, qk_norm="unit", gate="head", values_are_keys=True, sink=True, position=None,
                                   bias={"rows": m["bias_rows"], "far": m["bias_max"]})
        left, right = m["left"], m["right"]
        rot = left["rot"]
        attention = self._attention(left, pre + "left.", qk_norm="head", gate="channel", position=PartSpec(
            "rotary", {"theta": rot["base"], "head_dim": left["dim"], "dims": rot["dims"], "pairing": "half", "frequencies": "direct", "stretch": rot.get("scaling")}))
        state_space = PartSpec("state_space", {"prefix": pre + "right.", "hidden": self.width, "heads": right["heads"], "value_dim": right["vdim"], "state": right["state"],
                                               "groups": right["groups"], "taps": right["conv"], "norm_parts": right["norm_groups"], "eps": self.eps})
        return PartSpec("parallel", {"branches": (attention, state_space), "scales": (0.5, 0.5), "hidden": self.width,
                                     "norms": (pre + "left.out", pre + "right.out"), "eps": self.eps})

    def spec(self) -> ModelSpec:
        if self.wants_shapes():
            raise AlofaError("invalid_argument", "the rows of a bias table are not known yet: they come from the tensor's shape (sized_by) or the key bias_rows")
        h = self.width
        layers = []
        for i, l in enumerate(self.layers):
            p = f"l{i}."
            ff = None if l["mlp"] is None else PartSpec("dense_activated", {
                "prefix": p + "mlp.", "hidden": h, "intermediate": l["mlp"]["ff"], "activation": "gelu_tanh", "biases": True,
                "names": {"up": "up", "down": "down", "up_bias": "up.b", "down_bias": "down.b"}})
            subs = 1 if ff is None else 2
            layers.append(LayerSpec(prefix=p, block=PartSpec("scaled_prenorm", {"hidden": h, "residual_scale": 1.0, "channel_scales": tuple(p + f"ls{s + 1}" for s in range(subs))}),
                                    parts=dict(mixer=self._mixer_spec(l["type"], l["mixer"], p + "mix."), feed_forward=ff,
                                               norms=tuple(self._norm(p + f"norm{s + 1}") for s in range(subs)))))
        return ModelSpec(
            hidden_size=h, vocab_size=self.vocab, max_positions=1 << 30,
            embedding=PartSpec("token_embedding", {"name": "embed", "vocab": self.vocab, "width": h, "scale": self.embed_scale, "init": "unit"}),
            layers=tuple(layers), order=tuple(RunEntry(i) for i in range(len(layers))), final_norm=self._norm("final.norm"),
            head=PartSpec("lm_head", {"name": "head", "tied_to": None, "vocab": self.vocab, "width": h, "init": "fan_in"}))

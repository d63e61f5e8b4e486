"""Retotar: a decoder whose layers are listed one by one in config.json; every layer has one of three mixers (softmax attention within
a window whose heads talk after the softmax, a linear attention with a constant decay per head, a matrix memory with exponential gates)
and an optional mixture of experts; a norm stands in front of every sub-layer and another behind it.

config.json: ``architecture`` "Retotar"; ``vocab``, ``width``; ``norm.eps``; ``embedding.scale``; ``layers``: a list of {``type``,
``mixer``, ``mlp``}. Tensor names: ``embed``, ``l<i>.`` + ``norm1``/``norm1b``/``norm2``/``norm2b`` (+ ``.b``), ``mix.*``, ``mlp.*``;
``final.norm`` (+ ``.b``), ``head``.

The model: a token's row of ``embed`` times ``embedding.scale``. A layer: x += norm1b(mixer(norm1(x))), then, unless ``mlp`` is null,
x += norm2b(mlp(norm2(x))); all norms are layer norms with weight and bias. The logits are the head's product of the final norm's rows.

Mixers by ``type``:
  attention  ``heads`` query and ``kv_heads`` key/value heads of ``dim`` and ``vdim`` channels; rotary positions on the first ``rot.dims``
             channels of queries and keys (``rot.base``; every frequency divided by ``rot.scaling.factor``), which are then divided by their
             root mean square; values turned by their own positions over all their channels (``rot.base``, never scaled) and the heads'
             outputs turned back; scores times ``scale``; a row sees the last ``mask.size`` keys; the heads' softmax weights mixed by
             ``talk``; a sigmoid gate ``g``. With ``kv_from``: j the layer has no key and value projections and reads layer j's pages.
  lightning  ``heads`` x (``dim``, ``vdim``), q, k, v through silu, one ``decay`` per head, the heads normed together, a sigmoid gate.
  mlstm      ``heads`` x (``dim``, ``vdim``), log-space input and forget gates capped at ``gate_cap``, a running maximum that starts at 0.
The feed-forward (``mlp.kind`` "moe"): ``router.experts`` gated feed-forwards of ``expert.ff`` channels and ``router.identity`` experts
behind them that hand their input on; softmax scores over all of them; the choice by score + ``correction`` within the best
``router.groups.keep`` of ``router.groups.count`` groups of neighbours; a token takes ``router.top``, weighted by their scores."""
from __future__ import annotations

import copy
from dataclasses import dataclass

from ..config.base import LayerSpec, ModelConfig, ModelSpec, PartSpec, RunEntry
from ..errors import AlofaError
from .tugalix import _get, _positive

MIXERS = ("attention", "lightning", "mlstm")


def _attention(m: dict, where: str) -> dict:
    out = {k: _get(m, k, int, where) for k in ("heads", "kv_heads", "dim", "vdim")}
    _positive(where, **out)
    if out["heads"] % out["kv_heads"]:
        raise AlofaError("parse", "kv_heads must divide heads", f"heads={out['heads']} kv_heads={out['kv_heads']} config={where}")
    if out["vdim"] % 2:
        raise AlofaError("parse", "values are turned in pairs: vdim is even", f"vdim={out['vdim']} config={where}")
    out["scale"] = _get(m, "scale", float, where)
    rot = _get(m, "rot", dict, where)
    r = {"base": _get(rot, "base", float, where), "dims": _get(rot, "dims", int, where)}
    _positive(where, base=r["base"], dims=r["dims"])
    if r["dims"] % 2 or r["dims"] > out["dim"]:
        raise AlofaError("parse", "rot.dims is even and at most the head's size", f"dims={r['dims']} dim={out['dim']} config={where}")
    if rot.get("scaling") is not None:
        r["scaling"] = {"factor": _get(rot["scaling"], "factor", float, where)}
        _positive(where, factor=r["scaling"]["factor"])
    out["rot"] = r
    if m.get("mask") is not None:
        out["mask"] = {"size": _get(m["mask"], "size", int, where)}
        _positive(where, size=out["mask"]["size"])
    if m.get("kv_from") is not None:
        out["kv_from"] = _get(m, "kv_from", int, where)
    return out


def _recurrent(kind: str, m: dict, where: str) -> dict:
    out = {k: _get(m, k, int, where) for k in ("heads", "dim", "vdim")}
    _positive(where, **out)
    if kind == "lightning":
        out["decay"] = [float(x) for x in _get(m, "decay", list, where)]
        if len(out["decay"]) != out["heads"]:
            raise AlofaError("parse", "one decay per head", f"heads={out['heads']} decay={len(out['decay'])} config={where}")
    else:
        out["gate_cap"] = _get(m, "gate_cap", float, where)
        _positive(where, gate_cap=out["gate_cap"])
    return out


def _mlp(mlp, where: str):
    if mlp is None:
        return None
    if _get(mlp, "kind", str, where) != "moe":
        raise AlofaError("unsupported", "no such feed-forward in this design", f"kind={mlp['kind']} config={where}")
    r = _get(mlp, "router", dict, where)
    router = {"experts": _get(r, "experts", int, where), "top": _get(r, "top", int, where)}
    _positive(where, **router)
    router["identity"] = _get(r, "identity", int, where) if r.get("identity") is not None else 0
    if r.get("groups") is not None:
        router["groups"] = {"count": _get(r["groups"], "count", int, where), "keep": _get(r["groups"], "keep", int, where)}
        _positive(where, **router["groups"])
    groups = router.get("groups", {"count": 1, "keep": 1})
    routed = router["experts"] + router["identity"]
    if router["identity"] < 0 or routed % groups["count"] or groups["keep"] > groups["count"] or router["top"] > groups["keep"] * (routed // groups["count"]):
        raise AlofaError("parse", "equal groups of experts, of which the kept ones hold at least the experts a token takes",
                         f"experts={router['experts']} identity={router['identity']} groups={groups} top={router['top']} config={where}")
    ff = _get(_get(mlp, "expert", dict, where), "ff", int, where)
    _positive(where, ff=ff)
    return {"kind": "moe", "router": router, "expert": {"ff": ff}}


@dataclass(frozen=True)
class RetotarConfig(ModelConfig):
    vocab: int
    width: int
    eps: float
    embed_scale: float
    layers: tuple      # per layer a dict {type, mixer, mlp}, checked

    architecture = "Retotar"

    @classmethod
    def from_dict(cls, raw: dict, where: str = "<dict>") -> "RetotarConfig":
        layers = []
        for i, l in enumerate(_get(raw, "layers", list, where)):
            at = f"{where} layers[{i}]"
            kind = _get(l, "type", str, at)
            if kind not in MIXERS:
                raise AlofaError("unsupported", "no such mixer in this design", f"type={kind} known={','.join(MIXERS)} config={at}")
            m = _get(l, "mixer", dict, at)
            layers.append({"type": kind, "mixer": _attention(m, at) if kind == "attention" else _recurrent(kind, m, at), "mlp": _mlp(l.get("mlp"), at)})
        if not layers:
            raise AlofaError("parse", "a model has at least one layer", f"config={where}")
        for i, l in enumerate(layers):
            j = l["mixer"].get("kv_from") if l["type"] == "attention" else None
            if j is None:
                continue
            src = layers[j]["mixer"] if 0 <= j < i and layers[j]["type"] == "attention" else None
            if src is None or src.get("kv_from") is not None or any(src[k] != l["mixer"][k] for k in ("kv_heads", "dim", "vdim")):
                raise AlofaError("parse", "kv_from names an earlier attention layer with projections of its own and heads of the same sizes", f"layer={i} kv_from={j} config={where}")
        cfg = cls(vocab=_get(raw, "vocab", int, where), width=_get(raw, "width", int, where), eps=_get(_get(raw, "norm", dict, where), "eps", float, where),
                  embed_scale=_get(_get(raw, "embedding", dict, where), "scale", float, where), layers=tuple(layers))
        _positive(where, vocab=cfg.vocab, width=cfg.width, eps=cfg.eps)
        return cfg

    def to_dict(self) -> dict:
        return {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.eps},
                "embedding": {"scale": self.embed_scale}, "layers": copy.deepcopy(list(self.layers))}

    # ---- the model as data
    def _norm(self, name: str) -> PartSpec:
        return PartSpec("layernorm", {"name": name, "bias": name + ".b", "width": self.width, "eps": self.eps})

    def _kept(self, i: int):
        """How long layer i's keys are kept: the longest window among the layers that read them (None: for good)."""
        windows = [l["mixer"].get("mask", {}).get("size") if l["mixer"].get("mask") is not None else None
                   for j, l in enumerate(self.layers) if l["type"] == "attention" and (j == i or l["mixer"].get("kv_from") == i)]
        return None if any(w is None for w in windows) else max(windows)

    def _mixer_spec(self, i: int, kind: str, m: dict, pre: str) -> PartSpec:
        h = self.width
        if kind == "lightning":
            return PartSpec("lightning_attention", {"prefix": pre, "hidden": h, "heads": m["heads"], "key_dim": m["dim"], "value_dim": m["vdim"],
                                                    "decay": tuple(m["decay"]), "eps": self.eps})
        if kind == "mlstm":
            return PartSpec("matrix_memory", {"prefix": pre, "hidden": h, "heads": m["heads"], "key_dim": m["dim"], "value_dim": m["vdim"],
                                              "gate_cap": m["gate_cap"], "eps": self.eps})
        rot = m["rot"]
        source = m.get("kv_from")
        window = m["mask"]["size"] if m.get("mask") is not None else None
        return PartSpec("talking_attention", {
            "prefix": pre, "hidden": h, "heads": m["heads"], "kv_heads": m["kv_heads"], "head_dim": m["dim"], "v_head_dim": m["vdim"], "scale": m["scale"],
            "window": window, "keep_window": self._kept(i if source is None else source),
            "position": PartSpec("rotary", {"theta": rot["base"], "head_dim": rot["dims"], "factor": (rot.get("scaling") or {}).get("factor", 1.0)}),
            "value_position": PartSpec("rotary", {"theta": rot["base"], "head_dim": m["vdim"]}),
            "unit_norm": True, "eps": self.eps, "talk": True, "gate": True, "owns_cache": source is None})

    def _feed_forward(self, mlp, pre: str):
        if mlp is None:
            return None
        r = mlp["router"]
        return PartSpec("routed_experts", {
            "prefix": pre, "hidden": self.width, "experts": r["experts"], "top": r["top"], "score": "softmax", "correction": "correction",
            "groups": r.get("groups"), "passing": r["identity"], "renormalize": False, "expert": {"intermediate": mlp["expert"]["ff"]}, "shared": None,
            "activation": "silu_glu", "router_init": "decisive", "names": {"router": "router", "expert": "e{}", "shared": "shared", "gate": "gate", "up": "up", "down": "down"}})

    def spec(self) -> ModelSpec:
        h = self.width
        layers, order = [], []
        for i, l in enumerate(self.layers):
            p = f"l{i}."
            ff = self._feed_forward(l["mlp"], p + "mlp.")
            names = ("norm1", "norm1b") if ff is None else ("norm1", "norm1b", "norm2", "norm2b")
            layers.append(LayerSpec(prefix=p, block=PartSpec("sandwich", {"hidden": h}),
                                    parts=dict(mixer=self._mixer_spec(i, l["type"], l["mixer"], p + "mix."), feed_forward=ff, norms=tuple(self._norm(p + n) for n in names))))
            order.append(RunEntry(i, cache_of=l["mixer"].get("kv_from") if l["type"] == "attention" else None))
        return ModelSpec(
            hidden_size=h, vocab_size=self.vocab, max_positions=1 << 30,
            embedding=PartSpec("token_embedding", {"name": "embed", "vocab": self.vocab, "width": h, "scale": self.embed_scale, "init": "unit"}),
            layers=tuple(layers), order=tuple(order), final_norm=self._norm("final.norm"),
            head=PartSpec("lm_head", {"name": "head", "tied_to": None, "vocab": self.vocab, "width": h, "init": "fan_in"}))

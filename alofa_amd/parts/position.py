"""Position encodings.

Rotary: per position p and pair index i < d/2 the angle is p * theta^(-2i/d);
the pair (x[i], x[i + d/2]) of every query and key head is rotated by it. The
table is built once on the host exactly as the reference builds it: the inverse
frequency and the angle in float32, cos and sin evaluated in float64 and rounded
once (src/alofa/model/arch/qwen.mojo:830-880)."""
from __future__ import annotations

import math

import numpy as np
import torch

from ..config.base import PartSpec
from ..errors import AlofaError
from .base import PositionEncoding, register_part


class Rotary(PositionEncoding):
    """params: theta, head_dim, pairing ("half": channel i < dims/2 is paired with i + dims/2; "neighbours": channel 2i with
    2i + 1), dims (how many of a head's first channels are rotated, default all of them; the angle of pair i is
    p * theta^(-2i/dims), the channels from ``dims`` on pass unchanged), factor (every frequency is divided by it: positions
    stretched linearly; default 1), stretch ({factor, original, fast, slow}: frequencies stretched by wavelength: with
    dim(t) = dims ln(original / (2 pi t)) / (2 ln theta), lo = max(floor(dim(fast)), 0), hi = min(ceil(dim(slow)), dims - 1) and
    ramp_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1), pair i turns at f_i / factor * ramp_i + f_i (1 - ramp_i), and cos and sin
    are multiplied by 0.1 ln(factor) + 1), frequencies ("reciprocal": 1 / float32(theta^(2i/dims)) in float32, the default;
    "direct": theta^(-2i/dims) formed in float64 and rounded once).

    The kernels pair channel j with j + head_dim/2. With dims < head_dim the table holds the angle zero for the pairs
    beyond dims/2, and ``channel_order`` names the order of a head's channels in which the design's pairs lie that
    way: whoever projects queries and keys puts their channels in that order (both alike, so their products do not
    change)."""

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        self.theta = float(spec.params["theta"])
        self.head_dim = int(spec.params["head_dim"])
        self.dims = int(spec.params.get("dims") or self.head_dim)
        self.factor = float(spec.params.get("factor") or 1.0)
        if not self.factor > 0:
            raise AlofaError("invalid_argument", "the factor that stretches positions is positive", f"factor={self.factor}")
        if self.dims <= 0 or self.dims % 2 or self.dims > self.head_dim:
            raise AlofaError("unsupported", "rotated channels: an even count, at most the head's size", f"dims={self.dims} head_dim={self.head_dim}")
        self.pairing = spec.params.get("pairing", "half")
        if self.pairing not in ("half", "neighbours"):
            raise AlofaError("unsupported", "pairs are (j, j + dims/2) or (2j, 2j + 1)", f"pairing={spec.params['pairing']}")
        self.direct = spec.params.get("frequencies", "reciprocal") == "direct"
        self.stretch = spec.params.get("stretch")
        if self.stretch is not None:
            st = {k: float(self.stretch[k]) for k in ("factor", "original", "fast", "slow")}
            if not (st["factor"] > 0 and st["original"] > 0 and st["fast"] > 0 and st["slow"] > 0 and self.theta > 1):
                raise AlofaError("invalid_argument", "a stretch by wavelength takes positive numbers and a base above one", f"stretch={self.stretch} theta={self.theta}")
            self.stretch = st
        if self.head_dim <= 0 or self.head_dim % 2:
            raise AlofaError("unsupported", "head dimension must be positive and even", f"head_dim={self.head_dim}")

    def host_table(self, n_positions: int):
        half = self.head_dim // 2
        inv = np.zeros(half, dtype=np.float32)      # (pairs beyond dims/2 keep the angle zero: they pass unchanged)
        for i in range(self.dims // 2):
            if self.direct:
                inv[i] = np.float32(self._frequency(i))
                continue
            inv[i] = np.float32(1.0) / np.float32(math.pow(self.theta, (2.0 * i) / self.dims))
            if self.factor != 1.0:
                inv[i] = inv[i] / np.float32(self.factor)
        ang = np.arange(n_positions, dtype=np.float32)[:, None] * inv[None, :]
        ang = ang.astype(np.float32).astype(np.float64)
        cos, sin = np.cos(ang), np.sin(ang)
        if self.stretch is not None:      # (the pairs that are turned grow; the channels that pass stay as they are)
            mag = 0.1 * math.log(self.stretch["factor"]) + 1.0
            cos[:, :self.dims // 2] *= mag
            sin[:, :self.dims // 2] *= mag
        return cos.astype(np.float32), sin.astype(np.float32)

    def _frequency(self, i: int) -> float:
        """Pair i's frequency in float64, with the linear factor and the stretch by wavelength."""
        f = math.pow(self.theta, -2.0 * i / self.dims) / self.factor
        st = self.stretch
        if st is not None:
            def dim_of(turns):
                return self.dims * math.log(st["original"] / (2.0 * math.pi * turns)) / (2.0 * math.log(self.theta))
            lo = max(math.floor(dim_of(st["fast"])), 0)
            hi = min(math.ceil(dim_of(st["slow"])), self.dims - 1)
            ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
            f = f / st["factor"] * ramp + f * (1.0 - ramp)
        return f

    def channel_order(self):
        if self.dims == self.head_dim and self.pairing == "half":
            return None
        r, rest = self.dims // 2, (self.head_dim - self.dims) // 2
        if self.pairing == "neighbours":
            return [*range(0, self.dims, 2), *range(self.dims, self.dims + rest), *range(1, self.dims, 2), *range(self.dims + rest, self.head_dim)]
        return [*range(r), *range(self.dims, self.dims + rest), *range(r, self.dims), *range(self.dims + rest, self.head_dim)]

    @classmethod
    def for_head(cls, spec, head_dim: int):
        p = dict(spec.params)
        p["dims"] = int(p.get("dims") or p["head_dim"])
        p["head_dim"] = int(head_dim)
        return PartSpec(spec.kind, p)

    def table(self, n_positions: int):
        """One table per (theta, head size) serves every layer of the model (kept on the runtime).
        A table that has to grow is replaced; the old one is kept alive, since a captured graph
        may still read it (for positions it covers)."""
        key = ("rotary", self.theta, self.head_dim, self.dims, self.factor, self.direct, tuple(sorted(self.stretch.items())) if self.stretch else None)
        have = self.rt.shared.get(key)
        if have is None or have[0].shape[0] < n_positions:
            n = max(n_positions, 2 * have[0].shape[0] if have else 0)
            c, s = self.host_table(n)
            if have is not None:
                self.rt.shared.setdefault("retired tables", []).append(have)
            have = self.rt.shared[key] = (torch.from_numpy(c).to(self.rt.device), torch.from_numpy(s).to(self.rt.device))
        return have


class NoPosition(PositionEncoding):
    """No encoding: queries and keys are used as projected. Expressed as a
    rotation by angle zero so that the fused cache write serves it too.
    params: head_dim."""

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        self.head_dim = int(spec.params["head_dim"])

    def table(self, n_positions: int):
        key = ("no rotation", self.head_dim)
        have = self.rt.shared.get(key)
        if have is None or have[0].shape[0] < n_positions:
            half = self.head_dim // 2
            if have is not None:
                self.rt.shared.setdefault("retired tables", []).append(have)
            have = self.rt.shared[key] = (torch.ones(n_positions, half, dtype=torch.float32, device=self.rt.device),
                                          torch.zeros(n_positions, half, dtype=torch.float32, device=self.rt.device))
        return have


register_part("position", "rotary", Rotary)
register_part("position", "none", NoPosition)

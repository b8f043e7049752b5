"""Rotary position encoding (rotate-half): the frequencies, and the table of a step.

freq_i = theta^(-2i / rotary_dim) in float64 (src/model.rs:638-657); the table of a step is
(sin, cos)(pos * freq_i) computed in float64 on the device and rounded once to float32
(src/model.rs:2612-2621), shared by every layer whose encoding has the same parameters.
Parameters: `head_dim`, `rotary_dim` (the leading dims that rotate; the whole head here),
`theta`; optional `pairing` (which places make a pair: "halves", (i, i + rotary_dim / 2), the
default, or "neighbours", (2i, 2i + 1); the table is the same, the mixer's kernel applies it) and
`scaling`, a change of the frequencies for contexts longer than a model was trained on:

* {"kind": "stretch", factor, low, high, original}: by wavelength l = 2 pi / f against the
  original context: f is kept where l < original / high, divided by `factor` where
  l > original / low, and between the two blended with s = (original / l - low) / (high - low)
  as (1 - s) f / factor + s f;
* {"kind": "ramp", factor, original, fast, slow}: by pair index: with
  pair(t) = rotary_dim ln(original / (2 pi t)) / (2 ln theta), lo = max(floor(pair(fast)), 0),
  hi = min(ceil(pair(slow)), rotary_dim - 1) and r_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1)
  the frequency is r_i f_i / factor + (1 - r_i) f_i, and cos and sin are both multiplied by
  `magnitude` = 0.1 ln(factor) + 1, which the mixer's kernel applies.
"""
from __future__ import annotations

import math

import torch

from ..config.base import ConfigError
from .base import PositionEncoding, register_position


class RotaryEncoding(PositionEncoding):
    graph_safe = True
    def __init__(self, params, prefix=""):
        super().__init__(params, prefix)
        self.head_dim = int(params["head_dim"])
        self.rotary_dim = int(params.get("rotary_dim", self.head_dim))
        self.theta = float(params["theta"])
        if self.rotary_dim % 2 or not 0 < self.rotary_dim <= self.head_dim:
            raise ConfigError(f"rotary_dim {self.rotary_dim} must be even and at most head_dim {self.head_dim}")
        self.pairing = params.get("pairing", "halves")
        if self.pairing not in ("halves", "neighbours"):
            raise ConfigError(f"rotary pairing '{self.pairing}' is not known (halves, neighbours)")
        self.scaling = dict(params["scaling"]) if params.get("scaling") else None
        self.magnitude = 1.0
        if self.scaling is not None:
            kind = self.scaling.get("kind")
            if kind not in ("stretch", "ramp"):
                raise ConfigError(f"rotary scaling '{kind}' is not known (stretch, ramp)")
            if kind == "ramp":
                self.magnitude = 0.1 * math.log(float(self.scaling["factor"])) + 1.0
        self.key = None
        self._freqs = None

    def frequencies(self) -> torch.Tensor:
        n, dims = self.rotary_dim // 2, self.rotary_dim
        f = [self.theta ** (-2.0 * i / dims) for i in range(n)]
        sc = self.scaling
        if sc is not None and sc["kind"] == "stretch":
            factor, low, high, original = (float(sc[k]) for k in ("factor", "low", "high", "original"))
            for i, fi in enumerate(f):
                wavelength = 2.0 * math.pi / fi
                if wavelength > original / low:
                    f[i] = fi / factor
                elif wavelength >= original / high:
                    s = (original / wavelength - low) / (high - low)
                    f[i] = (1.0 - s) * fi / factor + s * fi
        elif sc is not None:
            factor, original, fast, slow = (float(sc[k]) for k in ("factor", "original", "fast", "slow"))
            pair_of = lambda turns: dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(self.theta))
            lo, hi = max(math.floor(pair_of(fast)), 0), min(math.ceil(pair_of(slow)), dims - 1)
            for i, fi in enumerate(f):
                ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
                f[i] = fi / factor * ramp + fi * (1.0 - ramp)
        return torch.tensor(f, dtype=torch.float64)

    def load(self, store, rt) -> None:
        f = self.frequencies()
        # encodings with the same frequencies share one table per step; a subclass that
        # changes the frequencies gets a table of its own
        self.key = ("rotary", tuple(f.tolist()))
        self._freqs = f.to(rt.device)

    def tables(self, ctx) -> torch.Tensor:
        """float32 [T, rotary_dim / 2, 2] for the positions of this step (made once per step)."""
        t = ctx.shared.get(self.key)
        if t is None:
            t = ctx.ws.take((ctx.n_tokens, self.rotary_dim // 2, 2), torch.float32)
            ctx.rt.k.rope_table(ctx.positions, self._freqs, t)
            ctx.shared[self.key] = t
        return t


register_position("rope", RotaryEncoding)

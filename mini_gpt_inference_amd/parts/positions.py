"""Position encodings.

A position encoding can act in two places: on the residual stream right after the
token embedding (`embedding_table`), or on queries and keys inside a mixer
(`rotate`).  A part implements the hooks it needs and leaves the others alone.
"""

from __future__ import annotations

import math
from typing import Dict, Optional

import torch

from .base import Part, StepContext, TABLE, WeightRequest, register_position


class PositionEncoding(Part):
    category = "position"
    max_positions: Optional[int] = None   # hard bound on positions, None = unbounded
    rotates = False                       # True if rotate() changes queries and keys

    def embedding_table(self) -> Optional[torch.Tensor]:
        """A [max_positions, width] table whose row pos[t] is added to token t's embedding."""
        return None

    def rotate(self, ctx: StepContext, q: torch.Tensor, k: torch.Tensor, n_tokens: int) -> None:
        """Acts on projected queries and keys in place, before the keys are cached."""
        return None


@register_position("learned_absolute")
class LearnedAbsolutePositions(PositionEncoding):
    """x0[t] += pos_emb[pos_t] with pos_t the absolute position, which must be < max_positions
    (reference: src/minigpt_infer/model.py:124,177-183)."""

    graph_safe = True

    plan_safe = True

    def __init__(self, max_positions: int, width: int) -> None:
        self.max_positions, self.width = int(max_positions), int(width)
        self.weight: Optional[torch.Tensor] = None

    def weight_requests(self) -> Dict[str, WeightRequest]:
        return {"weight": WeightRequest((self.max_positions, self.width), TABLE)}

    def embedding_table(self) -> Optional[torch.Tensor]:
        return self.weight


@register_position("none")
class NoPositions(PositionEncoding):
    """No position signal at all."""

    graph_safe = True

    plan_safe = True

    def __init__(self) -> None:
        pass


@register_position("rotary_half")
class RotaryHalf(PositionEncoding):
    """Rotation of queries and keys by position, on the first `dims` channels of every head:
    channel i is paired with channel i + dims/2, and at position p the pair (u, w) becomes
    (u cos a - w sin a, w cos a + u sin a) with a = p * f_i, f_i = base^(-2i/dims) / factor (factor: linear
    scaling of the positions).  The other channels pass unchanged.  A mixer that rotates owns one of
    these (its constants are the mixer's); the kernels that apply it take the frequency table.

    `scaling` changes the frequencies pair by pair, for contexts longer than the `original` one:
    - {"kind": "stretch", "factor", "low", "high", "original"}: by wavelength l = 2 pi / f.  f stays where
      l < original / high, becomes f / factor where l > original / low, and between the two
      (1 - s) f / factor + s f with s = (original / l - low) / (high - low);
    - {"kind": "ramp", "factor", "original", "fast", "slow"}: by pair index.  With
      at(t) = dims ln(original / (2 pi t)) / (2 ln base), lo = max(floor(at(fast)), 0),
      hi = min(ceil(at(slow)), dims - 1) and r_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1):
      f_i r_i / factor + f_i (1 - r_i); and every cosine and sine is multiplied by
      `magnitude` = 0.1 ln(factor) + 1."""

    graph_safe = True
    plan_safe = True
    rotates = True

    def __init__(self, dims: int, base: float, factor: float = 1.0, scaling: Optional[dict] = None) -> None:
        self.dims, self.base, self.factor = int(dims), float(base), float(factor)
        if self.dims <= 0 or self.dims % 2 or self.base <= 0.0 or self.factor <= 0.0:
            raise ValueError(f"rotation over {dims} channels with base {base} and factor {factor}")
        self.scaling = dict(scaling) if scaling else None
        self.magnitude = 1.0        # what every cosine and sine is multiplied by
        if self.scaling is not None:
            kind = self.scaling.get("kind")
            wanted = {"stretch": ("factor", "low", "high", "original"), "ramp": ("factor", "original", "fast", "slow")}
            if kind not in wanted or any(k not in self.scaling for k in wanted[kind]):
                raise ValueError(f"rotation scaling {scaling!r}: kind 'stretch' or 'ramp' with {wanted}")
            if not float(self.scaling["factor"]) > 0.0 or not float(self.scaling["original"]) > 0.0:
                raise ValueError("rotation scaling: factor and original must be positive")
            if kind == "ramp":
                if not (float(self.scaling["fast"]) > 0.0 and float(self.scaling["slow"]) > 0.0) or self.base == 1.0:
                    raise ValueError("rotation scaling: fast and slow must be positive, and the base not 1")
                self.magnitude = 0.1 * math.log(float(self.scaling["factor"])) + 1.0
        self._freq: Dict[torch.device, torch.Tensor] = {}

    def frequency_values(self) -> list:
        """The angle per position of every pair, in double precision."""
        plain = [self.base ** (-2.0 * i / self.dims) / self.factor for i in range(self.dims // 2)]
        sc = self.scaling
        if sc is None:
            return plain
        factor, original = float(sc["factor"]), float(sc["original"])
        if sc["kind"] == "stretch":
            low, high, out = float(sc["low"]), float(sc["high"]), []
            for f in plain:
                wavelength = 2.0 * math.pi / f
                if wavelength < original / high:
                    out.append(f)
                elif wavelength > original / low:
                    out.append(f / factor)
                elif high == low:      # (no wavelength lies between two equal bounds; one that sits on them counts as long)
                    out.append(f / factor)
                else:
                    s = (original / wavelength - low) / (high - low)
                    out.append((1.0 - s) * f / factor + s * f)
            return out
        at = lambda turns: self.dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(self.base))
        lo = max(math.floor(at(float(sc["fast"]))), 0)
        hi = min(math.ceil(at(float(sc["slow"]))), self.dims - 1)
        out = []
        for i, f in enumerate(plain):
            r = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
            out.append(f / factor * r + f * (1.0 - r))
        return out

    def frequencies(self, device: torch.device) -> torch.Tensor:
        """float32 [dims / 2]: the angle per position of every pair, computed in double precision."""
        f = self._freq.get(device)
        if f is None:
            f = torch.tensor(self.frequency_values(), dtype=torch.float64).to(torch.float32).to(device)
            self._freq[device] = f
        return f

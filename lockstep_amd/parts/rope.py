"""Rotary position encoding.  ``rope_half``: the pair of dimension ``i`` is
``i + rotary_dim/2``; ``rope_scaled`` adds a choice of the pairing and frequencies stretched by wavelength.  Tables are built in float64 on the host and kept in
float32, ``inv_freq[i] = theta^(-2i/rotary_dim)``, ``angle = position *
inv_freq`` (reference engine/model/qwen3.py:117-129).  The mixer applies them
inside its fused kernel."""

from __future__ import annotations

import torch

from ..config.base import PartSpec
from .base import PositionEncoding, bump_device_epoch, register_part

# Layers with the same constants share one pair of tables per device.
_TABLES: dict[tuple, list] = {}


@register_part("rope_half")
class RotaryHalf(PositionEncoding):
    """Parameters: ``rotary_dim`` (even, at most the head size), ``theta``."""

    graph_safe = True
    repeatable = True

    def __init__(self, spec: PartSpec, prefix: str = ""):
        super().__init__(spec, prefix)
        self.rotary_dim = int(spec["rotary_dim"])
        self.theta = float(spec["theta"])
        if self.rotary_dim % 2 or self.rotary_dim <= 0:
            raise ValueError(f"rotary_dim {self.rotary_dim} must be a positive even number")
        self._store = None

    @property
    def cos(self):
        return None if self._store is None else self._store[0]

    @property
    def sin(self):
        return None if self._store is None else self._store[1]

    def share_key(self):
        return (self.rotary_dim, self.theta)

    def tables(self, positions: torch.Tensor):
        half = self.rotary_dim // 2
        exponent = torch.arange(0, half, dtype=torch.float64) * 2.0 / self.rotary_dim
        inv_freq = 1.0 / (self.theta ** exponent)
        angles = positions.to(torch.float64)[:, None] * inv_freq[None, :]
        return angles.cos().to(torch.float32), angles.sin().to(torch.float32)

    def bind(self, rt) -> None:
        """Attach to the tables that all layers with these constants share on this device."""
        self._store = _TABLES.setdefault((self.rotary_dim, self.theta, str(rt.device)), [None, None])

    def ensure(self, max_position: int, rt) -> None:
        if self._store is None:
            self.bind(rt)
        have = 0 if self._store[0] is None else self._store[0].shape[0]
        if max_position <= have:
            return
        size = max(max_position, 2 * have, 256)
        cos, sin = self.tables(torch.arange(size))
        self._store[0] = cos.to(rt.device).contiguous()
        self._store[1] = sin.to(rt.device).contiguous()
        bump_device_epoch()


@register_part("rope_scaled")
class RotaryScaled(RotaryHalf):
    """Rotary encoding with a choice of which dimensions form a pair and with frequencies that are
    stretched by wavelength.  Parameters: ``rotary_dim`` (even), ``theta``, ``pairing`` (``"half"``:
    dimension ``i`` with ``i + rotary_dim/2``; ``"neighbours"``: ``2i`` with ``2i + 1``) and ``scaling``
    (None, or ``factor``, ``low``, ``high``, ``original``): with the wavelength ``l = 2 pi / f`` of a
    pair's frequency ``f = theta^(-2i/rotary_dim)``, ``f`` stays where ``l < original/high``, becomes
    ``f / factor`` where ``l > original/low``, and in between is ``(1 - s) f / factor + s f`` with
    ``s = (original/l - low) / (high - low)``.

    Kernels that know ``neighbours`` rotate such pairs in place; for those that pair ``i`` with
    ``i + rotary_dim/2`` only, ``dim_order`` states the reordering of a head that brings the pairs there."""

    def __init__(self, spec: PartSpec, prefix: str = ""):
        super().__init__(spec, prefix)
        self.pairing = str(spec.params.get("pairing", "half"))
        if self.pairing not in ("half", "neighbours"):
            raise ValueError(f"pairing {self.pairing!r} is not one of half, neighbours")
        scaling = spec.params.get("scaling")
        self.scaling = None
        if scaling:
            self.scaling = tuple(float(scaling[key]) for key in ("factor", "low", "high", "original"))
            factor, low, high, original = self.scaling
            if not (factor > 0 and original > 0 and high > low >= 0):
                raise ValueError(f"frequency scaling needs factor > 0, original > 0 and high > low >= 0, got {scaling}")

    @property
    def neighbours(self) -> bool:
        return self.pairing == "neighbours"

    def share_key(self):
        return (self.rotary_dim, self.theta, self.scaling)      # (the pairing does not enter the tables)

    def frequencies(self) -> torch.Tensor:
        import math

        half = self.rotary_dim // 2
        exponent = torch.arange(0, half, dtype=torch.float64) * 2.0 / self.rotary_dim
        freq = 1.0 / (self.theta ** exponent)
        if self.scaling is None:
            return freq
        factor, low, high, original = self.scaling
        wavelength = 2.0 * math.pi / freq
        blend = (original / wavelength - low) / (high - low)
        mixed = (1.0 - blend) * freq / factor + blend * freq
        return torch.where(wavelength * high < original, freq, torch.where(wavelength * low > original, freq / factor, mixed))

    def tables(self, positions: torch.Tensor):
        angles = positions.to(torch.float64)[:, None] * self.frequencies()[None, :]
        return angles.cos().to(torch.float32), angles.sin().to(torch.float32)

    def bind(self, rt) -> None:
        self._store = _TABLES.setdefault((self.rotary_dim, self.theta, self.scaling, str(rt.device)), [None, None])

    def dim_order(self, head_dim: int):
        if not self.neighbours:
            return None
        return list(range(0, self.rotary_dim, 2)) + list(range(1, self.rotary_dim, 2)) + list(range(self.rotary_dim, head_dim))


@register_part("rope_ramped")
class RotaryRamped(RotaryScaled):
    """Rotary encoding whose frequencies are stretched along a ramp over the pair index, and whose cosines
    and sines are enlarged.  Parameters: ``rotary_dim``, ``theta``, ``pairing`` and ``scaling`` (None, or
    ``factor``, ``original``, ``fast``, ``slow``).  With ``c(t) = rotary_dim ln(original / (2 pi t)) / (2 ln
    theta)``, the pair index at which a rotation makes ``t`` turns within ``original`` positions, ``lo =
    max(floor(c(fast)), 0)`` and ``hi = min(ceil(c(slow)), rotary_dim - 1)``: pair ``i`` has the frequency
    ``f_i / factor * r_i + f_i (1 - r_i)`` with ``r_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1)``, and
    both tables are multiplied by ``0.1 ln(factor) + 1``."""

    def __init__(self, spec: PartSpec, prefix: str = ""):
        scaling = spec.params.get("scaling")
        super().__init__(PartSpec(spec.kind, {**spec.params, "scaling": None}), prefix)
        self.spec = spec
        self.ramp = None
        if scaling:
            self.ramp = tuple(float(scaling[key]) for key in ("factor", "original", "fast", "slow"))
            factor, original, fast, slow = self.ramp
            if not (factor > 0 and original > 0 and fast > 0 and slow > 0 and self.theta > 1):
                raise ValueError(f"a frequency ramp needs positive factor, original, fast and slow and theta > 1, got {scaling}")

    def share_key(self):
        return (self.rotary_dim, self.theta, "ramp", self.ramp)

    def magnitude(self) -> float:
        import math

        return 1.0 if self.ramp is None else 0.1 * math.log(self.ramp[0]) + 1.0

    def frequencies(self) -> torch.Tensor:
        import math

        half = self.rotary_dim // 2
        index = torch.arange(0, half, dtype=torch.float64)
        freq = 1.0 / (self.theta ** (index * 2.0 / self.rotary_dim))
        if self.ramp is None:
            return freq
        factor, original, fast, slow = self.ramp

        def pair_of(turns: float) -> float:
            return self.rotary_dim * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(self.theta))

        lo = max(math.floor(pair_of(fast)), 0)
        hi = min(math.ceil(pair_of(slow)), self.rotary_dim - 1)
        ramp = ((index - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
        return freq / factor * ramp + freq * (1.0 - ramp)

    def tables(self, positions: torch.Tensor):
        angles = positions.to(torch.float64)[:, None] * self.frequencies()[None, :]
        scale = self.magnitude()
        return (angles.cos() * scale).to(torch.float32), (angles.sin() * scale).to(torch.float32)

    def bind(self, rt) -> None:
        self._store = _TABLES.setdefault((self.rotary_dim, self.theta, "ramp", self.ramp, str(rt.device)), [None, None])


@register_part("no_position")
class NoPosition(PositionEncoding):
    """Leaves queries and keys as they are."""

    graph_safe = True
    repeatable = True

    rotary_dim = 0
    cos = None
    sin = None

    def share_key(self):
        return ("none",)

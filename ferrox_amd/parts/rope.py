"""Rotary position encodings.  The attention kernels rotate q and k themselves
while they write the cache, so these parts only carry the constants.

'rope_neox' pairs (i, i + rot/2) — the layout of ferrox-core/src/attention.rs:20-32,
which the reference's registry gives this architecture
(ferrox-models/src/capability.rs:252-258); 'rope_interleaved' pairs (2i, 2i+1)
(attention.rs `apply_rope_interleaved`).  angle = pos * theta^(-2i/rot).
"""
from __future__ import annotations

from .base import POSITION_ENCODINGS, PositionEncoding, Rotary


class _Rotary(PositionEncoding):
    interleaved = False

    def __init__(self, head_dim: int, theta: float, rotary_dim: int | None = None):
        self.head_dim = int(head_dim)
        self.theta = float(theta)
        self.rotary_dim = int(rotary_dim if rotary_dim is not None else head_dim)
        if self.rotary_dim % 2 or not 0 <= self.rotary_dim <= self.head_dim:
            raise ValueError(f"rotary_dim {self.rotary_dim} must be even and at most head_dim {self.head_dim}")
        if not self.theta > 0:
            raise ValueError(f"rope theta must be positive, got {self.theta}")

    def rotary(self):
        return Rotary(self.rotary_dim, self.theta, self.interleaved)


@POSITION_ENCODINGS.register("rope_neox")
class NeoxRope(_Rotary):
    interleaved = False


@POSITION_ENCODINGS.register("rope_interleaved")
class InterleavedRope(_Rotary):
    interleaved = True


@POSITION_ENCODINGS.register("none")
class NoPositions(PositionEncoding):
    def __init__(self, head_dim: int = 0):
        self.head_dim = head_dim

    def rotary(self):
        return Rotary(0, 1.0)


def scaled_frequencies(rotary_dim: int, theta: float, scaling) -> tuple:
    """theta^(-2i/rotary_dim) with a wavelength-dependent correction, in float64.  `scaling` = (factor, low, high,
    original): with L = 2 pi / f the wavelength of a pair, f is kept where L < original / high, divided by `factor`
    where L > original / low, and blended in between, (1 - s) f / factor + s f with
    s = (original / L - low) / (high - low): short waves keep their resolution, long ones are stretched to a
    context `factor` times the original one."""
    import math
    out = []
    for i in range(rotary_dim // 2):
        f = float(theta) ** (-2.0 * i / rotary_dim)
        if scaling is not None:
            factor, low, high, original = (float(x) for x in scaling)
            wavelength = 2.0 * math.pi / f
            if wavelength > original / low:
                f = f / factor
            elif wavelength >= original / high:
                s = (original / wavelength - low) / (high - low)
                f = (1.0 - s) * f / factor + s * f
        out.append(f)
    return tuple(out)


@POSITION_ENCODINGS.register("rope_scaled")
class ScaledRope(_Rotary):
    """A rotation whose frequencies are a table of this part's own (`scaled_frequencies`); either pairing."""

    def __init__(self, head_dim: int, theta: float, rotary_dim: int | None = None, interleaved: bool = False,
                 scaling=None):
        super().__init__(head_dim, theta, rotary_dim)
        self.interleaved = bool(interleaved)
        if scaling is not None:
            scaling = tuple(float(x) for x in scaling)
            if len(scaling) != 4 or min(scaling) <= 0 or not scaling[2] > scaling[1]:
                raise ValueError(f"rope scaling is (factor, low, high, original), all positive, high > low; got {scaling}")
        self.scaling = scaling
        self.frequencies = scaled_frequencies(self.rotary_dim, self.theta, scaling)

    def rotary(self):
        return Rotary(self.rotary_dim, self.theta, self.interleaved, None, self.frequencies)


def ramped_frequencies(rotary_dim: int, theta: float, factor: float, original: float, fast: float, slow: float) -> tuple:
    """theta^(-2i/rotary_dim) stretched by pair index, in float64.  d(t) = rotary_dim ln(original / (2 pi t)) /
    (2 ln theta) is the (fractional) pair whose wave makes t turns over `original` positions.  Pairs up to
    lo = max(floor(d(fast)), 0) keep their frequency f, pairs from hi = min(ceil(d(slow)), rotary_dim - 1) on get
    f / factor, and between them the two are blended with a ramp (i - lo) / max(hi - lo, 0.001) clamped to [0, 1]."""
    import math

    def pair_of(turns: float) -> float:
        return rotary_dim * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(theta))

    lo = max(math.floor(pair_of(fast)), 0)
    hi = min(math.ceil(pair_of(slow)), rotary_dim - 1)
    out = []
    for i in range(rotary_dim // 2):
        f = float(theta) ** (-2.0 * i / rotary_dim)
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(f / factor * ramp + f * (1.0 - ramp))
    return tuple(out)


@POSITION_ENCODINGS.register("rope_ramped")
class RampedRope(_Rotary):
    """A rotation for contexts `factor` times longer than the `original` one: frequencies stretched by pair index
    (`ramped_frequencies`), and cosine and sine both multiplied by 0.1 ln(factor) + 1, which makes up for the
    scores' loss of contrast under the slower waves.  `scaling` = (factor, original, fast, slow) or None (a plain
    rotation, magnitude 1).  Either pairing."""
    MAGNITUDE_SLOPE = 0.1

    def __init__(self, head_dim: int, theta: float, rotary_dim: int | None = None, interleaved: bool = False,
                 scaling=None):
        import math
        super().__init__(head_dim, theta, rotary_dim)
        self.interleaved = bool(interleaved)
        self.magnitude = 1.0
        if scaling is not None:
            scaling = tuple(float(x) for x in scaling)
            if len(scaling) != 4 or min(scaling) <= 0 or self.theta == 1.0:
                raise ValueError(f"ramped rope scaling is (factor, original, fast, slow), all positive, theta not 1; got {scaling}")
            self.frequencies = ramped_frequencies(self.rotary_dim, self.theta, *scaling) if self.rotary_dim else ()
            self.magnitude = self.MAGNITUDE_SLOPE * math.log(scaling[0]) + 1.0
        else:
            self.frequencies = tuple(self.theta ** (-2.0 * i / self.rotary_dim) for i in range(self.rotary_dim // 2))
        self.scaling = scaling

    def rotary(self):
        return Rotary(self.rotary_dim, self.theta, self.interleaved, None, self.frequencies, self.magnitude)

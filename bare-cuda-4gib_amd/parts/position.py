"""Position encodings applied to queries and keys before keys are cached."""
from __future__ import annotations

import math

from ..errors import ConfigError
from .base import Part, register_part


class Rotary(Part):
    """Rotary positions with the rotate-half pairing (element i with element
    i + dim/2): inv_freq_i = theta^(-2i/dim), angle = position * inv_freq_i,
    (lo, hi) -> (lo cos - hi sin, hi cos + lo sin), angles in float
    (reference: engine/kernels/rope.cu:44-53).  ``dim`` may be smaller than the
    head size; the remaining elements pass through.

    ``scaling`` (factor F, original L, fast, slow) stretches the slow pairs for contexts beyond L: with
    e(t) = dim ln(L / (2 pi t)) / (2 ln theta), lo = max(floor(e(fast)), 0), hi = min(ceil(e(slow)), dim - 1) and
    r_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1), pair i turns with inv_freq_i / F * r_i + inv_freq_i (1 - r_i), and
    cosines and sines are multiplied by 0.1 ln F + 1.  The kernels that rotate inside a product take no scaling
    (``fused()`` is None then); ``table(ctx)`` gives every row's cosines and sines to whoever rotates by a table.

    A ``scaling`` that gives (factor F, original L, low, high) instead goes by r_i = L inv_freq_i / (2 pi), the turns a pair
    makes over L positions: above ``high`` the pair turns as it is, below ``low`` with inv_freq_i / F, and from low to high with
    inv_freq_i (s + (1 - s) / F), s = (r_i - low) / (high - low); cosines and sines keep their size.

    ``pairing`` "neighbours" turns element 2i with element 2i + 1 instead (the same angles, the same table); only
    kernels that rotate by a table know that pairing."""
    category = "position"
    graph_safe = True     # launches kernels only: may run inside a captured graph

    def __init__(self, theta: float, dim: int, scaling=None, pairing: str = "half"):
        if pairing not in ("half", "neighbours"):
            raise ConfigError(f"rotary: pairing must be 'half' or 'neighbours', got {pairing!r}")
        self.pairing = pairing
        if dim <= 0 or dim % 2:
            raise ConfigError(f"rotary: dim must be positive and even, got {dim}")
        if theta <= 0:
            raise ConfigError(f"rotary: theta must be positive, got {theta}")
        self.theta, self.dim = float(theta), int(dim)
        self.scaling = None
        self.by_wavelength = False
        if scaling is not None:
            self.by_wavelength = isinstance(scaling, dict) and "low" in scaling and "high" in scaling
            keys = ("factor", "original", "low", "high") if self.by_wavelength else ("factor", "original", "fast", "slow")
            try:
                self.scaling = tuple(float(scaling[k]) for k in keys)
            except (KeyError, TypeError, ValueError):
                raise ConfigError(f"rotary: scaling must give {', '.join(keys)}, got {scaling!r}") from None
            if min(self.scaling) <= 0 or (self.theta == 1.0 and not self.by_wavelength):
                raise ConfigError(f"rotary: scaling {scaling!r} with theta {theta}: every number must be positive, theta not 1")
            if self.by_wavelength and self.scaling[2] == self.scaling[3]:
                raise ConfigError(f"rotary: scaling {scaling!r}: low and high must differ")
        self._freqs = None

    def fused(self):
        return (self.dim, self.theta) if self.scaling is None and self.pairing == "half" else None

    @property
    def neighbours(self) -> bool:
        return self.pairing == "neighbours"

    def apply(self, qkv, ctx, n_heads, n_kv_heads, head_dim):
        raise ConfigError("rotary: scaled frequencies and neighbouring pairs are applied by a table (table(ctx)); this mixer "
                          "rotates inside its product")

    def frequencies(self):
        """(what pair i turns by per position, for i < dim / 2, as Python floats; the factor on cosines and sines)."""
        half = self.dim // 2
        freqs = [self.theta ** (-2.0 * i / self.dim) for i in range(half)]
        if self.scaling is None:
            return freqs, 1.0
        if self.by_wavelength:
            factor, original, low, high = self.scaling
            out = []
            for f in freqs:
                wavelength = 2.0 * math.pi / f
                if wavelength > original / low:
                    f = f / factor
                elif wavelength >= original / high:
                    s = (original / wavelength - low) / (high - low)
                    f = (1.0 - s) * f / factor + s * f
                out.append(f)
            return out, 1.0
        factor, original, fast, slow = self.scaling
        where = lambda t: self.dim * math.log(original / (2.0 * math.pi * t)) / (2.0 * math.log(self.theta))      # noqa: E731
        lo, hi = max(math.floor(where(fast)), 0), min(math.ceil(where(slow)), self.dim - 1)
        ramp = [min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0) for i in range(half)]
        return [f / factor * r + f * (1.0 - r) for f, r in zip(freqs, ramp)], 0.1 * math.log(factor) + 1.0

    def table(self, ctx):
        """[T, dim / 2, 2] float32: every row's cosines and sines, made once a step for all layers that rotate alike."""
        import torch
        from ..csrc import ops
        freqs, amplitude = self.frequencies()
        if self._freqs is None or self._freqs.device != ctx.positions.device:
            self._freqs = torch.tensor(freqs, dtype=torch.float64, device=ctx.positions.device)
        return ctx.shared(("rotary_table", self.dim, self.theta, self.scaling, self.by_wavelength),
                          lambda: ops.rotary_table(ctx.positions, self._freqs, amplitude))


class NoPosition(Part):
    """No position encoding: queries and keys are used as projected."""
    category = "position"
    graph_safe = True     # launches kernels only: may run inside a captured graph

    def fused(self):
        return 0, 1.0


register_part("position", "rotary", Rotary)
register_part("position", "none", NoPosition)

"""Position encodings for a mixer's queries and keys.

Rotary: pair (i, i + rotary_dim/2) of a head is rotated by the angle
pos * theta^(-2i/rotary_dim), the rotate-half pairing of the reference's kernel
(orchestrator/kernels.py:264-297).  The cache stores keys after rotation, so an
encoding must be a function of the absolute position alone.
"""
from __future__ import annotations

import math

import numpy as np

from ..runtime.device import Tensor
from .base import Part, register_part


class Rotary(Part):
    graph_safe = True      # its launches take what changes from step to step from device memory alone

    def __init__(self, spec):
        if spec.rotary_dim % 2 or not (0 < spec.rotary_dim <= spec.head_dim):
            raise ValueError(f"rotary_dim must be even and in (0, head_dim], got {spec.rotary_dim}")
        if getattr(spec, "linear_factor", None) is not None and not spec.linear_factor > 0:
            raise ValueError(f"linear_factor must be positive, got {spec.linear_factor}")
        ws = getattr(spec, "wavelength_scaling", None)
        if ws is not None and not (ws[0] > 0 and ws[3] > 0 and ws[1] > 0 and ws[2] > ws[1]):
            raise ValueError(f"wavelength_scaling needs factor, original > 0 and high > low > 0, got {ws}")
        self.spec = spec
        self.inv_freq = None

    def frequencies(self) -> np.ndarray:
        s = self.spec
        i = np.arange(s.rotary_dim // 2, dtype=np.float64)
        f = 1.0 / np.power(float(s.theta), 2.0 * i / s.rotary_dim)
        scaling = getattr(s, "scaling", None)
        if scaling is not None:
            # pair numbers at which `fast` and `slow` turns fit into `original` positions bound a
            # ramp; below it a frequency stays, above it is divided by the factor
            factor, original, fast, slow = (float(v) for v in scaling)
            at = lambda turns: s.rotary_dim * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(float(s.theta)))
            lo = max(math.floor(at(fast)), 0)
            hi = min(math.ceil(at(slow)), s.rotary_dim - 1)
            ramp = np.clip((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
            f = f / factor * ramp + f * (1.0 - ramp)
        linear = getattr(s, "linear_factor", None)
        if linear is not None:
            f = f / float(linear)
        by_wavelength = getattr(s, "wavelength_scaling", None)
        if by_wavelength is not None:
            # each frequency on its own, by how its wavelength compares with the original length
            factor, low, high, original = (float(v) for v in by_wavelength)
            for n in range(len(f)):
                length = 2.0 * math.pi / f[n]
                if length > original / low:
                    f[n] = f[n] / factor
                elif length >= original / high:
                    share = (original / length - low) / (high - low)
                    f[n] = (1.0 - share) * f[n] / factor + share * f[n]
        return f.astype(np.float32)

    def magnitude(self) -> float:
        """What sines and cosines are multiplied by (1 without frequency scaling)."""
        scaling = getattr(self.spec, "scaling", None)
        return 0.1 * math.log(float(scaling[0])) + 1.0 if scaling is not None else 1.0

    @property
    def interleaved(self) -> bool:
        return bool(getattr(self.spec, "interleaved", False))

    def load(self, weights, rt, dtype):
        self.inv_freq = rt.upload(self.frequencies())

    def rotary_tables(self):
        return self.inv_freq, self.spec.rotary_dim

    def apply(self, ctx, qkv: Tensor, num_heads: int, num_kv_heads: int, head_dim: int):
        raise NotImplementedError("a rotary encoding is applied by the mixer's fused kernel")


class NoPosition(Part):
    graph_safe = True      # its launches take what changes from step to step from device memory alone

    def __init__(self, spec):
        self.spec = spec

    def rotary_tables(self):
        return None

    def apply(self, ctx, qkv, num_heads, num_kv_heads, head_dim):
        return None


register_part("position", "rotary", Rotary)
register_part("position", "none", NoPosition)

"""Rotary position encoding: float32 tables built on the CPU.

inv_freq[i] = 1 / theta**(2i/rot_dim) is computed on the CPU in float32 with the
positive exponent and a reciprocal, and the angle is float32(position) * inv_freq
(qil/model.py:99-108).  Computing theta**(-e), or computing on the GPU, crosses
bfloat16 rounding edges of cos/sin (docs/OPTIMIZATION_DEBUG_LOG.md:23-33).  The
tables stay float32 whatever the model's dtype.  Pairing is (i, i + rot_dim/2)
(qil/model.py:42-46).
"""
import math

import torch

from .base import PositionEncoding, Rotation


class Rotary(PositionEncoding):
    def __init__(self, head_dim, theta, max_positions, *, rot_dim=None, device='cpu'):
        super().__init__()
        self.head_dim, self.theta, self.max_positions = int(head_dim), float(theta), int(max_positions)
        self.rot_dim = self.head_dim if rot_dim is None else int(rot_dim)
        if self.rot_dim % 2 or not 0 < self.rot_dim <= self.head_dim:
            raise ValueError('rot_dim must be even and at most head_dim')
        self.device = device
        self._rotation = None

    def angles(self, positions):
        exponent = torch.arange(0, self.rot_dim, 2, device='cpu', dtype=torch.float32) / self.rot_dim
        inv_freq = 1.0 / (self.theta ** exponent)
        return positions.to('cpu', torch.float32)[:, None] * inv_freq[None, :]

    def rotation(self):
        if self._rotation is None:
            angles = self.angles(torch.arange(self.max_positions))
            self._rotation = Rotation(angles.cos().to(self.device).contiguous(),
                                      angles.sin().to(self.device).contiguous(), self.rot_dim)
        return self._rotation


class RotaryFrequencies(PositionEncoding):
    """The rotation as its frequencies alone: f_i = base**(-2 i / rot_dim), i < rot_dim / 2, made in float64 and held
    in float32.  Kernels that take it make the angle position * f_i and its cosine and sine themselves, in float32,
    so no table bounds the positions.  Pairing is (i, i + rot_dim / 2).

    ``scaling`` (factor, low, high, original): long waves are slowed.  With the wavelength l = 2 pi / f, f stays where
    l < original / high, becomes f / factor where l > original / low, and between the two is
    (1 - s) f / factor + s f with s = (original / l - low) / (high - low)."""

    def __init__(self, rot_dim, base, *, device='cpu', scaling=None):
        super().__init__()
        self.rot_dim, self.base, self.device = int(rot_dim), float(base), device
        self.scaling = None if scaling is None else tuple(float(v) for v in scaling)
        if self.scaling is not None and (len(self.scaling) != 4 or not all(v > 0 for v in self.scaling) or
                                         not self.scaling[2] > self.scaling[1]):
            raise ValueError('scaling is (factor, low, high, original), all positive, high above low')
        if self.rot_dim < 2 or self.rot_dim % 2:
            raise ValueError('rot_dim must be even and at least 2')
        if not self.base > 0:
            raise ValueError('the base must be positive')
        self._frequencies = None

    def rotation(self):
        return Rotation(None, None, self.rot_dim, self.frequencies())

    def _scaled(self, f):
        if self.scaling is None:
            return f
        factor, low, high, original = self.scaling
        wavelength = 2.0 * math.pi / f
        if wavelength < original / high:
            return f
        if wavelength > original / low:
            return f / factor
        s = (original / wavelength - low) / (high - low)
        return (1.0 - s) * f / factor + s * f

    def frequencies(self):
        if self._frequencies is None:
            values = [self._scaled(self.base ** (-2.0 * i / self.rot_dim)) for i in range(self.rot_dim // 2)]
            self._frequencies = torch.tensor(values, dtype=torch.float64).to(torch.float32).to(self.device).contiguous()
        return self._frequencies

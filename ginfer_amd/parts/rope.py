"""Rotary position encoding, NeoX pairing (j, j + rotary_dim/2)."""
import torch

from .base import Part
from .registry import register_position


@register_position("rope_neox")
class RotaryNeoX(Part):
    """Tables sin/cos[p, j] of angle (float)p * inv_freq[j], inv_freq[j] = 1 / theta^(j / half), all in
    32-bit as the reference builds them (ginfer/core/op/kernels/cuda/rope_kernel.cu:13-16 and :61-72),
    computed once on the host and uploaded.  The rotation itself is part of the mixer's kernel
    (ginfer/core/op/kernels/cuda/rope_kernel.cu:83-102)."""

    capturable = True

    style = "neox"

    def __init__(self, theta, rotary_dim, max_positions, dtype=None, device=None, scaling=None, wide_frequencies=False,
                 linear_factor=None):
        """wide_frequencies: the frequencies are worked out in 64-bit and rounded to 32-bit once (else every step of
        their formula is 32-bit, as the reference has it).  scaling: None, or dict(factor, low, high, original): frequencies rescaled by their wavelength l = 2 pi / f
        (the scheme of the Llama 3.1 models): kept where l < original / high, divided by `factor` where l > original /
        low, and between the two blended with s = (original / l - low) / (high - low): (1 - s) f / factor + s f.
        linear_factor: every frequency is divided by it (positions stretched evenly), worked out in 64-bit."""
        if rotary_dim % 2 or rotary_dim <= 0:
            raise ValueError("rotary_dim must be positive and even, got %r" % (rotary_dim,))
        self.theta, self.rotary_dim, self.max_positions = float(theta), int(rotary_dim), int(max_positions)
        self.linear_factor = None if linear_factor is None else float(linear_factor)
        if self.linear_factor is not None and not self.linear_factor > 0:
            raise ValueError("linear_factor must be positive, got %r" % (linear_factor,))
        self.wide_frequencies = bool(wide_frequencies) or scaling is not None or self.linear_factor is not None
        self.scaling = None if scaling is None else {k: float(scaling[k]) for k in ("factor", "low", "high", "original")}
        if self.scaling is not None and not (self.scaling["high"] > self.scaling["low"] > 0 and self.scaling["factor"] > 0
                                             and self.scaling["original"] > 0):
            raise ValueError("frequency scaling needs factor > 0, original > 0 and high > low > 0, got %r" % (scaling,))
        self.device = device
        self._tables = None
        self._limit = None

    def limit_positions(self, n):
        """Tables need not be longer than the longest sequence the engine will hold."""
        self._limit = min(self.max_positions, int(n))
        self._tables = None

    @property
    def num_positions(self):
        return self._limit or self.max_positions

    def _wide_frequencies(self, half):
        """The frequencies theta^(-j / half), rescaled by wavelength where the part has a scaling; worked out in 64-bit,
        handed on in 32-bit."""
        import math
        sc = self.scaling
        out = []
        for j in range(half):
            f = self.theta ** (-float(j) / half)
            wavelength = 2.0 * math.pi / f
            if sc is None:
                pass
            elif wavelength > sc["original"] / sc["low"]:
                f = f / sc["factor"]
            elif wavelength >= sc["original"] / sc["high"]:
                s = (sc["original"] / wavelength - sc["low"]) / (sc["high"] - sc["low"])
                f = (1.0 - s) * f / sc["factor"] + s * f
            if self.linear_factor is not None:
                f = f / self.linear_factor
            out.append(f)
        return torch.tensor(out, dtype=torch.float64).to(torch.float32)

    def tables(self):
        """(cos, sin), float32 [num_positions, rotary_dim / 2] on the device."""
        if self._tables is None:
            half = self.rotary_dim // 2
            j = torch.arange(half, dtype=torch.float32)
            inv_freq = 1.0 / torch.pow(torch.tensor(self.theta, dtype=torch.float32), j / float(half))
            if self.wide_frequencies:
                inv_freq = self._wide_frequencies(half)
            p = torch.arange(self.num_positions, dtype=torch.float32)
            ang = p[:, None] * inv_freq[None, :]
            self._tables = (torch.cos(ang).to(self.device).contiguous(), torch.sin(ang).to(self.device).contiguous())
        return self._tables


@register_position("rope_interleaved")
class RotaryInterleaved(RotaryNeoX):
    """The same angles and tables; the mixer's kernel turns the neighbouring coordinates (2j, 2j + 1) by angle j, where the
    NeoX pairing turns (j, j + rotary_dim / 2)."""

    style = "interleaved"

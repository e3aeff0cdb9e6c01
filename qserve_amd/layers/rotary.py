"""Rotary position tables: plain, with YaRN frequency scaling, or with piecewise (wavelength-band) frequency scaling.

Rotation of pair i at position p by the angle a = p * f_i: (u cos a - v sin a, v cos a + u sin a), f_i = base^(-2i / dims).
Which two dimensions form pair i is the kernels' business (neighbours 2i, 2i + 1, or halves i, i + dims / 2): the table holds
cos and sin per (position, pair) and serves both.  With scaling {factor, original, fast, slow} (YaRN): the
dimension at which a wave makes t turns over the original context is c(t) = dims * ln(original / (2 pi t)) / (2 ln base);
between lo = max(floor(c(fast)), 0) and hi = min(ceil(c(slow)), dims - 1) a linear ramp r_i blends the interpolated
frequency f_i / factor (r = 1) with the plain one (r = 0), and cos and sin carry the magnitude 0.1 ln(factor) + 1.

With scaling {factor, original, low, high} (bands of wavelength l_i = 2 pi / f_i): l_i < original / high keeps f_i,
l_i > original / low uses f_i / factor, and between the two s = (original / l_i - low) / (high - low) blends
(1 - s) f_i / factor + s f_i; the magnitude stays 1.

The table is made on the host in float64 (angles exact to the last bit a float holds) and kept on the device as float
[positions, 2, dims / 2] (cos, then sin); it grows when a longer position is asked for.
"""
import math

import torch


class RotaryTable:
    def __init__(self, dims, base, scaling=None, device="cpu", positions=4096):
        if dims <= 0 or dims % 2:
            raise ValueError(f"rotary dims must be even and positive, not {dims}")
        self.dims, self.base, self.scaling, self.device = int(dims), float(base), scaling, device
        half = self.dims // 2
        f = torch.tensor([self.base ** (-2.0 * i / self.dims) for i in range(half)], dtype=torch.float64)
        self.magnitude = 1.0
        if scaling and "low" in scaling:
            factor, orig, low, high = (float(scaling[k]) for k in ("factor", "original", "low", "high"))
            out = []
            for fi in f.tolist():
                wavelength = 2.0 * math.pi / fi
                if wavelength < orig / high:
                    out.append(fi)
                elif wavelength > orig / low:
                    out.append(fi / factor)
                else:
                    s = (orig / wavelength - low) / (high - low)
                    out.append((1.0 - s) * fi / factor + s * fi)
            f = torch.tensor(out, dtype=torch.float64)
        elif scaling:
            factor, orig = float(scaling["factor"]), float(scaling["original"])

            def turns_dim(t):
                return self.dims * math.log(orig / (2.0 * math.pi * t)) / (2.0 * math.log(self.base))

            lo = max(math.floor(turns_dim(float(scaling["fast"]))), 0)
            hi = min(math.ceil(turns_dim(float(scaling["slow"]))), self.dims - 1)
            ramp = torch.tensor([min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0) for i in range(half)], dtype=torch.float64)
            f = f / factor * ramp + f * (1.0 - ramp)
            self.magnitude = 0.1 * math.log(factor) + 1.0
        self.freq = f
        self.table = None
        self.reserve(positions)

    def key(self):
        s = self.scaling
        return (self.dims, self.base, None if not s else tuple(sorted((k, float(v)) for k, v in s.items())))

    def reserve(self, positions):
        """Make the table cover positions [0, positions); returns it."""
        if self.table is None or self.table.size(0) < positions:
            n = max(int(positions), 1 if self.table is None else 2 * self.table.size(0))
            a = torch.arange(n, dtype=torch.float64)[:, None] * self.freq[None, :]
            t = torch.stack([torch.cos(a), torch.sin(a)], dim=1) * self.magnitude
            self.table = t.to(torch.float32).to(self.device).contiguous()
        return self.table

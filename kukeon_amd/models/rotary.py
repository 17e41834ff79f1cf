"""Rotary angle tables.

`angle_table` covers plain rotary frequencies and the YaRN rescaling of
them: frequencies whose wavelength exceeds the original context are divided
by `factor`, short wavelengths are kept, and a linear ramp over the pair
index blends the two; cos and sin are then scaled by 0.1 ln(factor) + 1.
Angles are formed in float64 and the table is stored in fp32, one row per
position: [cos_0 .. cos_(n-1) | sin_0 .. sin_(n-1)] with n = dims / 2.
"""
from __future__ import annotations

import math
from typing import Optional

import torch


def pair_frequencies(dims: int, base: float,
                     scaling: Optional[dict] = None):
    """-> (freq [dims/2] float64, amplitude) for pair i = dims 2i, 2i+1."""
    n = dims // 2
    i = torch.arange(n, dtype=torch.float64)
    f = torch.pow(torch.tensor(float(base), dtype=torch.float64),
                  -2.0 * i / dims)
    amp = 1.0
    if scaling:
        factor = float(scaling["factor"])
        orig = float(scaling["original"])

        def pair_of(turns: float) -> float:
            # pair index whose wavelength makes `turns` rotations over
            # the original context
            return dims * math.log(orig / (2.0 * math.pi * turns)) / \
                (2.0 * math.log(base))

        lo = max(math.floor(pair_of(float(scaling["fast"]))), 0)
        hi = min(math.ceil(pair_of(float(scaling["slow"]))), dims - 1)
        ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
        f = f / factor * ramp + f * (1.0 - ramp)
        amp = 0.1 * math.log(factor) + 1.0
    return f, amp


def angle_table(positions: int, dims: int, base: float,
                scaling: Optional[dict] = None) -> torch.Tensor:
    f, amp = pair_frequencies(dims, base, scaling)
    ang = torch.arange(positions, dtype=torch.float64)[:, None] * f[None, :]
    return torch.cat([ang.cos() * amp, ang.sin() * amp], dim=1).float()

"""Rotary position encoding with half-split pairing (i, i + r/2):
a = pos * theta^(-2i/r); (y_i, y_{i+r/2}) = (x_i cos a - x_{i+r/2} sin a,
x_i sin a + x_{i+r/2} cos a); dims >= r pass through
(reference: kernels/attention.cu:516-558; r = 2*floor(hd*partial/2),
kernels/register_kernels.cpp:702-704). The frequencies are computed once in
float64 and held in float32; the angle and its sine/cosine are formed in fp32
inside the fused q/k kernel from each row's own position.

Options of the same part: `rotary_dim` names the rotated dims outright; `interleaved` pairs dim
2i with 2i + 1 instead of i with i + r/2; `scaling` = {"kind": "yarn", factor, original, fast,
slow} stretches the slow frequencies for contexts longer than `original` positions: with
dim(t) = r ln(original / (2 pi t)) / (2 ln theta), lo = max(floor(dim(fast)), 0),
hi = min(ceil(dim(slow)), r - 1) and ramp_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1), frequency
i becomes f_i / factor * ramp_i + f_i (1 - ramp_i), and cos and sin are both multiplied by
0.1 ln(factor) + 1 (`mscale`; the rotated pairs grow by that factor)."""
from __future__ import annotations

import math

import torch

from .base import BuildEnv, PositionEncoding, param, register_part


@register_part("position", "rotary")
class Rotary(PositionEncoding):
    def __init__(self, params: dict, prefix: str, env: BuildEnv):
        super().__init__(prefix, env)
        self.head_dim = param(params, "head_dim", int)
        self.theta = param(params, "theta", float)
        partial = param(params, "partial_rotary_factor", float, 1.0)
        r = 2 * int(self.head_dim * partial / 2)
        self.rotary_dim = param(params, "rotary_dim", int, self.head_dim if r <= 0 else r)
        if self.rotary_dim % 2 or not 0 < self.rotary_dim <= self.head_dim:
            raise ValueError(f"rotary: rotary_dim {self.rotary_dim} must be even, positive and at most head_dim")
        self.interleaved = param(params, "interleaved", bool, False)
        r = self.rotary_dim
        i = torch.arange(0, r, 2, dtype=torch.float64)
        inv = 1.0 / (torch.tensor(self.theta, dtype=torch.float64) ** (i / r))
        scaling = param(params, "scaling", dict, None)
        if scaling is not None:
            kind = scaling.get("kind", "yarn")
            if kind != "yarn":
                raise ValueError(f"rotary: unknown scaling '{kind}'")
            factor, original = float(scaling["factor"]), float(scaling["original"])
            if factor <= 0 or original <= 0 or self.theta <= 1:
                raise ValueError("rotary: yarn scaling needs factor > 0, original > 0 and theta > 1")

            def dim_of(turns: float) -> float:
                return r * math.log(original / (2 * math.pi * turns)) / (2 * math.log(self.theta))

            lo = max(math.floor(dim_of(float(scaling["fast"]))), 0)
            hi = min(math.ceil(dim_of(float(scaling["slow"]))), r - 1)
            ramp = ((torch.arange(r // 2, dtype=torch.float64) - lo) / max(hi - lo, 0.001)).clamp(0, 1)
            inv = inv / factor * ramp + inv * (1 - ramp)
            self.mscale = 0.1 * math.log(factor) + 1.0
        self.inv_freq = inv.to(torch.float32).to(env.device).contiguous()

    def rotary(self):
        return self.inv_freq, self.rotary_dim


@register_part("position", "none")
class NoPosition(PositionEncoding):
    """No encoding of positions at this place."""

    def __init__(self, params: dict, prefix: str, env: BuildEnv):
        super().__init__(prefix, env)

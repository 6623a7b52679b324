"""Rotary position encoding, rotate-half pairing (flow_engine/model.py:26-33).

inv_freq[j] = theta^(-2j/rot) is computed on the host in float32 exactly as the
reference writes it; angles, cos and sin are float32 on the device, once per
step for all layers that share this part. `rotary_dim` < head_dim rotates only
the first rotary_dim elements of each head.

`stretch` = (factor, original context, fast, slow) stretches the encoding for
contexts beyond the one a model was trained on (YaRN: Peng et al., "YaRN:
Efficient Context Window Extension of Large Language Models"): with
pair(t) = rot * ln(original / (2 pi t)) / (2 ln theta), lo = max(floor(pair(fast)), 0),
hi = min(ceil(pair(slow)), rot - 1) and ramp_j = clamp((j - lo) / max(hi - lo, 0.001), 0, 1),
pair j turns with inv_freq[j] * (ramp_j / factor + 1 - ramp_j): pairs that turn
often within the original context keep their frequency, slow ones are divided by
the factor; cos and sin are both multiplied by 0.1 ln(factor) + 1.
"""
from __future__ import annotations

import math

import torch

from ..kernels import ops
from .base import PositionEncoding


class RotaryEmbedding(PositionEncoding):
    def __init__(self, head_dim, theta, rotary_dim=None, pairing="half", stretch=None):
        if pairing not in ("half", "adjacent"):
            raise ValueError("pairing must be 'half' or 'adjacent'")
        self.pairing = pairing
        self.head_dim = int(head_dim)
        self.theta = float(theta)
        self.rotary_dim = int(rotary_dim if rotary_dim is not None else head_dim)
        if self.rotary_dim % 2 or not 0 < self.rotary_dim <= self.head_dim:
            raise ValueError("rotary_dim must be even and at most head_dim")
        self.stretch = tuple(float(v) for v in stretch) if stretch else None
        if self.stretch and (len(self.stretch) != 4 or self.stretch[0] <= 0 or min(self.stretch[1:]) <= 0 or self.theta <= 1):
            raise ValueError("stretch is (factor, original context, fast, slow), all positive, with theta > 1")
        self.magnitude = 0.1 * math.log(self.stretch[0]) + 1.0 if self.stretch else 1.0
        self.inv_freq = None

    def frequencies(self):
        """The pairs' frequencies, float32 [rotary_dim / 2] on the host."""
        rot = self.rotary_dim
        if not self.stretch:
            return self.theta ** (-torch.arange(0, rot, 2, dtype=torch.float32) / rot)
        factor, original, fast, slow = self.stretch
        j = torch.arange(rot // 2, dtype=torch.float64)
        inv = self.theta ** (-2.0 * j / rot)

        def pair(turns):
            return rot * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(self.theta))
        lo, hi = max(math.floor(pair(fast)), 0), min(math.ceil(pair(slow)), rot - 1)
        ramp = ((j - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
        return (inv / factor * ramp + inv * (1.0 - ramp)).to(torch.float32)

    def bind(self, tensors, dtype, device):
        self.inv_freq = self.frequencies().to(device)          # a constant the tables are derived from, not a weight

    def tables(self, ctx):
        """(cos, sin), float32 [n_tokens, rotary_dim / 2], computed once per step."""
        key = ("rotary", id(self))
        hit = ctx.shared.get(key)
        if hit is None:
            half = self.rotary_dim // 2
            cos = ctx.scratch(f"rotary.cos.{id(self)}", (ctx.n_tokens, half), torch.float32)
            sin = ctx.scratch(f"rotary.sin.{id(self)}", (ctx.n_tokens, half), torch.float32)
            ops.rope_table(ctx.positions[0], self.inv_freq, cos, sin, self.magnitude)
            hit = ctx.shared[key] = (cos, sin)
        return hit


class NoPositionEncoding(PositionEncoding):
    """Mixers given this part rotate nothing."""
    rotary_dim = 0

    def tables(self, ctx):
        return None, None

"""Retention: linear attention with a fixed decay per head, no softmax and no denominator.

    q, k [heads x dim], v [heads x value_dim] from one packed product, q and k rotated, k times dim^-1/2
    S_t = decay_h S_(t-1) + k_t v_t^T,   o_t = S_t^T q_t          (S float32 [dim, value_dim] per head and request)
    out = W_o [ .. o_t,h / rms(o_t,h) * silu(g_t,h) .. ]           (g from the same packed product)

The state S is the mixer's whole memory: a fixed-size float32 state in its cache slot, zero when a request opens,
read at the start of a step's rows of a sequence and written at their end by the same workgroup. Rotation, the
decays, the state and all products with it are float32 in both precisions.
"""
from __future__ import annotations

import torch

from ..cache.spec import CacheNeed, FixedState
from ..kernels import ops
from .base import Mixer
from .linear import Linear


def _round_up(v, m):
    return (int(v) + m - 1) // m * m


class Retention(Mixer):
    STATE = "retention.s"

    def __init__(self, prefix, hidden, heads, dim, value_dim, decay, position, eps, names=("q", "k", "v", "g", "o"),
                 suffix=""):
        """decay: one factor per head; position: a rotary encoding over at most `dim` elements ('half' pairing) or a
        `NoPositionEncoding`; eps: of the per-head unit norm."""
        self.prefix, self.names = prefix, tuple(names)
        self.hidden, self.heads, self.dim, self.value_dim = int(hidden), int(heads), int(dim), int(value_dim)
        self.decay_values = [float(v) for v in decay]
        if len(self.decay_values) != self.heads:
            raise ValueError("one decay per head is needed")
        if not 1 <= self.dim <= 256:
            raise ValueError("the retention kernels take key sizes up to 256")
        if position.rotary_dim > self.dim or (position.rotary_dim and position.pairing != "half"):
            raise ValueError("the rotary encoding must cover at most dim elements with the 'half' pairing")
        self.position, self.eps = position, float(eps)
        # sizes on the device: tails of zeros (zero rows in the matrices), which add nothing to a product
        self.dim_dev, self.value_dev = _round_up(dim, 16), _round_up(value_dim, 16)
        kd, vd = (self.dim, self.dim_dev), (self.value_dim, self.value_dev)
        self.proj = Linear([prefix + n for n in self.names[:4]], hidden,
                           [heads * dim, heads * dim, heads * value_dim, heads * value_dim],
                           pad_out=[kd, kd, vd, vd], suffixes=(suffix, ".bias"))
        self.o = Linear([prefix + self.names[4]], heads * value_dim, [hidden], pad_in=vd, suffixes=(suffix, ".bias"))
        self.decay = None

    def parts(self):
        return [self.proj, self.o, self.position]

    def tensor_specs(self):
        return self.proj.tensor_specs() + self.o.tensor_specs()

    def bind(self, tensors, dtype, device):
        self.proj.bind(tensors, dtype, device)
        self.o.bind(tensors, dtype, device)
        self.position.bind(tensors, dtype, device)
        self.decay = torch.tensor(self.decay_values, dtype=torch.float32, device=device)   # constants of the configuration

    def cache_need(self):
        return CacheNeed(states=((self.STATE, FixedState((self.heads, self.dim_dev, self.value_dev), "float32")),))

    def forward(self, ctx, run, h, x, accumulate=True):
        n, H, Dp, Ep = ctx.n_tokens, self.heads, self.dim_dev, self.value_dev
        proj = ctx.scratch("retention.proj", (n, 2 * H * (Dp + Ep)))
        self.proj.forward(ctx, h, proj)
        cos, sin = self.position.tables(ctx)
        result = ctx.scratch("retention.o", (n, H * Ep), torch.float32)
        state = ctx.cache.states[run.cache_slot][self.STATE]
        common = (proj, 0, H * Dp, 2 * H * Dp, cos, sin, self.decay, state, ctx.q_start, ctx.state_slots)
        if ctx.n_decode:         # one-token sequences walk token by token
            ops.retention(*common, 0, ctx.n_decode, result, self.dim ** -0.5)
        portions = ctx.n_seqs - ctx.n_decode
        if portions:             # prompt portions in chunks on the matrix unit, long ones cut into segments
            floats = ops.retention_workspace_floats(portions, ctx.max_q_len, H, Dp, Ep)
            ws = ctx.workspace.get("retention.segments", (floats,), torch.float32) if floats else None
            ops.retention(*common, ctx.n_decode, portions, result, self.dim ** -0.5, max_q_len=ctx.max_q_len, workspace=ws)
        act = ctx.scratch("retention.act", (n, H * Ep))
        ops.unit_gate(result, proj[:, 2 * H * Dp + H * Ep:], act, H, self.value_dim, Ep, self.eps)
        if ctx.defer_sums and self.o.deferrable(n):
            return self.o.forward_partials(ctx, act, "o")          # whoever norms next adds them up
        self.o.forward(ctx, act, x, residual=x if accumulate else None)
        return None

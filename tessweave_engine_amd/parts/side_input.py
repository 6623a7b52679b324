"""A per-layer input from the token itself: each layer owns a slice of a second, narrow embedding table.

    e = table[token][layer * dim : (layer + 1) * dim]
    g = gelu_tanh(gate x) * e              (gate: [dim, hidden], x the residual stream)
    y = proj g                             (proj: [hidden, dim])
    x <- x + mult * y / sqrt(mean(y^2) + eps) * weight

The unit norm and the addition run in the kernel that ends a layer (`ops.layer_end`); this part
computes y in float32. The table is shared by all layers and bound once.
"""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.spec import MATRIX, NORMAL, ONE_PLUS_NORMAL, VECTOR, TensorSpec
from .base import Part
from .linear import Linear


class SideTable(Part):
    """The narrow embedding table [vocab, layers * dim] all layers' side inputs read."""

    def __init__(self, name, vocab, columns):
        self.name, self.vocab, self.columns = name, int(vocab), int(columns)
        self.weight = None

    def tensor_specs(self):
        return [TensorSpec(self.name, (self.vocab, self.columns), MATRIX, NORMAL)]

    def bind(self, tensors, dtype, device):
        self.weight = tensors.pop(self.name).contiguous()


class TokenSideInput(Part):
    def __init__(self, prefix, table, layer, hidden, dim, eps, names=("gate", "proj", "norm"), owns_table=False):
        """table: the `SideTable` all layers share; exactly one layer's part lists it as its own (owns_table)."""
        self.owns_table = bool(owns_table)
        self.table, self.layer, self.hidden, self.dim, self.eps = table, int(layer), int(hidden), int(dim), float(eps)
        self.gate = Linear([prefix + names[0]], hidden, [dim], suffixes=("", ".b"))
        self.proj = Linear([prefix + names[1]], dim, [hidden], suffixes=("", ".b"))
        self.norm_name = prefix + names[2]
        self.weight = None

    def parts(self):
        return [self.gate, self.proj] + ([self.table] if self.owns_table else [])

    def tensor_specs(self):
        return (self.table.tensor_specs() if self.owns_table else []) + self.gate.tensor_specs() + self.proj.tensor_specs() + \
            [TensorSpec(self.norm_name, (self.hidden,), VECTOR, ONE_PLUS_NORMAL)]

    def bind(self, tensors, dtype, device):
        if self.owns_table:
            self.table.bind(tensors, dtype, device)
        self.gate.bind(tensors, dtype, device)
        self.proj.bind(tensors, dtype, device)
        self.weight = tensors.pop(self.norm_name).contiguous()

    def weight_tensors(self):
        return [self.weight]

    def forward(self, ctx, x):
        """y float32 [n, hidden] for the residual stream x; the caller norms and adds it."""
        n = x.shape[0]
        rounded = ctx.scratch("side.x", (n, self.hidden))
        ops.round_rows(x, rounded)
        pre = ctx.scratch("side.pre", (n, self.dim), torch.float32)
        self.gate.forward(ctx, rounded, pre)
        g = ctx.scratch("side.g", (n, self.dim))
        ops.token_gate(pre, self.table.weight, ctx.token_ids, self.layer * self.dim, g, feed=ctx.token_feed)
        y = ctx.scratch("side.y", (n, self.hidden), torch.float32)
        self.proj.forward(ctx, g, y)
        return y

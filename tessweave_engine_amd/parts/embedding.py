"""Token embedding and the output head (flow_engine/model.py:100,108-112,176,204).

The embedding is a row gather without scaling, into the float32 residual
stream. The head multiplies the normalised rows that were asked for by its
matrix and returns float32 logits; a tied head uses the embedding's matrix and
its own checkpoint key is accepted but never required.
"""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.spec import MATRIX, NORMAL, TensorSpec
from .base import Part


class TokenEmbedding(Part):
    def __init__(self, name, vocab, hidden, suffix=".weight"):
        self.name, self.vocab, self.hidden = name, int(vocab), int(hidden)
        self.suffix = suffix
        self.weight = None

    def tensor_specs(self):
        return [TensorSpec(self.name + self.suffix, (self.vocab, self.hidden), MATRIX, NORMAL)]

    def bind(self, tensors, dtype, device):
        self.weight = tensors.pop(self.name + self.suffix).contiguous()

    def forward(self, ctx):
        x = ctx.scratch("residual", (ctx.n_tokens, self.hidden), torch.float32)
        return ops.embed_gather(ctx.token_ids, self.weight, x, feed=ctx.token_feed)


class PositionedEmbedding(TokenEmbedding):
    """Token embedding plus a learned vector per position (not scaled): x = table[token] + positions[p].

    `keep` = (workspace tag, leading size): the sum is also written to the first rows of entry 0 of the float32
    scratch buffer [leading, largest step's rows, hidden] of that tag, for models whose later layers read the
    embedding output again."""

    def __init__(self, name, vocab, hidden, position_name, max_positions, suffix=".weight", keep=None):
        super().__init__(name, vocab, hidden, suffix)
        self.position_name, self.max_positions, self.keep = position_name, int(max_positions), keep
        self.positions = None

    def tensor_specs(self):
        return super().tensor_specs() + [TensorSpec(self.position_name + self.suffix, (self.max_positions, self.hidden),
                                                    MATRIX, NORMAL)]

    def bind(self, tensors, dtype, device):
        super().bind(tensors, dtype, device)
        self.positions = tensors.pop(self.position_name + self.suffix).contiguous()

    def forward(self, ctx):
        x = super().forward(ctx)
        copy = None
        if self.keep is not None:
            tag, leading = self.keep
            copy = ctx.workspace.get(tag, (leading, ctx.max_tokens, self.hidden), torch.float32)[0, :ctx.n_tokens]
        return ops.add_table_rows(x, self.positions, ctx.positions[0], copy=copy)


class OutputHead(Part):
    def __init__(self, name, vocab, hidden, tied_to=None, suffix=".weight"):
        self.name, self.vocab, self.hidden = name, int(vocab), int(hidden)
        self.suffix = suffix
        self.tied_to = tied_to
        self.weight = None

    def tensor_specs(self):
        if self.tied_to is not None:
            return [TensorSpec(self.name + self.suffix, (self.vocab, self.hidden), MATRIX, NORMAL,
                               optional_alias_of=self.tied_to.name + self.tied_to.suffix)]
        return [TensorSpec(self.name + self.suffix, (self.vocab, self.hidden), MATRIX, NORMAL)]

    def bind(self, tensors, dtype, device):
        # The head's matrix is kept in the matrix kernels' shuffled layout; a tied head makes its own
        # shuffled copy of the embedding (the gather reads rows, the head streams MFMA blocks).
        source = self.tied_to.weight if self.tied_to is not None else tensors.pop(self.name + self.suffix).contiguous()
        if torch.device(device).type == "cuda" and ops.can_shuffle(source):
            self.weight = ops.shuffle_weight(source)
        else:
            self.weight = source

    def matrix(self):
        return self.weight

    def weight_tensors(self):
        return [self.weight]          # (the embedding's table is not listed by its part: a step gathers a few rows of it)

    def forward(self, ctx, h):
        # The logits live in a shared scratch buffer: they are valid until the next step.
        logits = ctx.workspace.get("logits", (h.shape[0], self.vocab), torch.float32)
        return ops.linear(h, self.matrix(), logits)

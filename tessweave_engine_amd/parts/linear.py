"""A linear layer over one or several checkpoint matrices with the same input.

Several matrices are packed by exact row concatenation into one weight, as the
reference packs q,k,v and gate,up (flow_engine/model.py:58-65): 7 matrix
products per layer become 4. `packed=False` keeps them apart (the reference's
`--unfused` ablation, cli.py:73); each then writes its own column range.
"""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.spec import MATRIX, VECTOR, NORMAL, TensorSpec
from .base import Part


def pad_groups(t, dim, unit, to):
    """T with every group of UNIT consecutive entries along DIM followed by TO - UNIT zeros."""
    if to == unit:
        return t
    shape = list(t.shape)
    groups = shape[dim] // unit
    out = t.new_zeros(shape[:dim] + [groups, to] + shape[dim + 1:])
    out.narrow(dim + 1, 0, unit).copy_(t.reshape(shape[:dim] + [groups, unit] + shape[dim + 1:]))
    return out.reshape(shape[:dim] + [groups * to] + shape[dim + 1:])


class Linear(Part):
    def __init__(self, names, in_features, out_features, bias=False, packed=True, glu=False,
                 pad_out=None, pad_in=None, suffixes=(".weight", ".bias")):
        """names[i] is the checkpoint prefix of the i-th matrix ("...q_proj"), out_features[i] its rows.

        glu: the two matrices are a gate and an up projection; if they can be packed with their
        rows interleaved (`gated` is then true after bind), `forward_glu` gives silu(gate) * up.
        pad_out = (unit, to): on the device every group of `unit` output rows (a head) is followed by
        `to - unit` rows of zeros (and zero biases), so the layer's output has groups of `to` columns
        whose tail is exactly zero. pad_in = (unit, to): the same for groups of input columns (the
        input then has groups of `to` columns, whose tails meet zeros). The checkpoint's tensors keep
        their own shapes. pad_out may also be a list with one (unit, to) or None per matrix, and pad_in a
        list of (columns, unit, to) runs that together cover the input (several inputs side by side, each
        with its own groups).
        bias may be a list with one flag per matrix: a matrix without one gets zeros on the device.
        suffixes: what a matrix's name is followed by in the checkpoint for its weight and its bias.
        """
        self.names = list(names)
        self.in_features = int(in_features)
        self.out_features = [int(o) for o in out_features]
        self.bias_flags = [bool(b) for b in bias] if isinstance(bias, (list, tuple)) else [bool(bias)] * len(self.names)
        if len(self.bias_flags) != len(self.names):
            raise ValueError("one bias flag per matrix is needed")
        self.has_bias = any(self.bias_flags)
        self.suffixes = tuple(suffixes)
        self.packed = bool(packed)
        self.glu = bool(glu)

        def pair(p):
            return tuple(int(v) for v in p) if p and p[0] != p[1] else None
        if pad_out and isinstance(pad_out[0], (list, tuple, type(None))):
            self.pad_outs = [pair(p) for p in pad_out]
        else:
            self.pad_outs = [pair(pad_out)] * len(self.names)
        if len(self.pad_outs) != len(self.names):
            raise ValueError("one output padding per matrix is needed")
        self.pad_out = self.pad_outs[0] if len(set(self.pad_outs)) == 1 else None
        if pad_in and isinstance(pad_in[0], (list, tuple)):
            self.pad_ins = [tuple(int(v) for v in run) for run in pad_in]
            if sum(run[0] for run in self.pad_ins) != self.in_features:
                raise ValueError("the input's padded runs must cover its columns")
            if all(u == t for _, u, t in self.pad_ins):
                self.pad_ins = None
        else:
            single = pair(pad_in)
            self.pad_ins = [(self.in_features, *single)] if single else None
        self.pad_in = pair(pad_in) if not (pad_in and isinstance(pad_in[0], (list, tuple))) else None
        for pad, rows in zip(self.pad_outs, self.out_features):
            if pad and (pad[1] < pad[0] or rows % pad[0]):
                raise ValueError("padded groups must divide the layer's sizes and may only grow")
        for columns, unit, to in self.pad_ins or []:
            if to < unit or columns % unit:
                raise ValueError("padded groups must divide the layer's sizes and may only grow")
        self.gated = False
        self.weights = []       # one tensor if packed, else one per name
        self.biases = []
        self._ws_floats = {}

    @property
    def total_out(self):
        return sum(self.out_features)

    def tensor_specs(self):
        specs = []
        for name, rows, flag in zip(self.names, self.out_features, self.bias_flags):
            specs.append(TensorSpec(name + self.suffixes[0], (rows, self.in_features), MATRIX, NORMAL))
            if flag:
                specs.append(TensorSpec(name + self.suffixes[1], (rows,), VECTOR, NORMAL))
        return specs

    @property
    def device_in(self):
        """Input columns on the device (padded groups included)."""
        if not self.pad_ins:
            return self.in_features
        return sum(columns // unit * to for columns, unit, to in self.pad_ins)

    @property
    def device_out(self):
        """Output columns of each matrix on the device (padded groups included)."""
        return [rows // pad[0] * pad[1] if pad else rows for rows, pad in zip(self.out_features, self.pad_outs)]

    def bind(self, tensors, dtype, device):
        weights = [tensors.pop(name + self.suffixes[0]) for name in self.names]
        biases = []
        if self.has_bias:
            biases = [tensors.pop(name + self.suffixes[1]) if flag else
                      torch.zeros(rows, dtype=torch.float32, device=weights[0].device)
                      for name, rows, flag in zip(self.names, self.out_features, self.bias_flags)]
        weights = [pad_groups(w, 0, *pad) if pad else w for w, pad in zip(weights, self.pad_outs)]
        biases = [pad_groups(b, 0, *pad) if pad else b for b, pad in zip(biases, self.pad_outs)]
        if self.pad_ins:
            padded = []
            for w in weights:
                runs, col = [], 0
                for columns, unit, to in self.pad_ins:
                    runs.append(pad_groups(w[:, col:col + columns], 1, unit, to))
                    col += columns
                padded.append(torch.cat(runs, 1) if len(runs) > 1 else runs[0])
            weights = padded
        self.gated = (self.glu and self.packed and len(weights) == 2 and
                      weights[0].shape == weights[1].shape and weights[0].shape[0] % 16 == 0)
        if self.gated:
            weights = [ops.interleave_glu_rows(*weights)]
            biases = [ops.interleave_glu_rows(*biases)] if biases else []
        elif self.packed and len(weights) > 1:
            weights = [torch.cat(weights, 0)]
            biases = [torch.cat(biases, 0)] if biases else []
        # On a GPU the matrices are kept in the kernels' shuffled layout (an exact permutation)
        # whenever their rows are a multiple of 16 bytes; otherwise row-major for the generic kernel.
        on_gpu = torch.device(device).type == "cuda"
        self.weights = [ops.shuffle_weight(w.contiguous()) if on_gpu and ops.can_shuffle(w) else w.contiguous()
                        for w in weights]
        self.biases = [b.contiguous() for b in biases]
        del weights, biases

    def weight_tensors(self):
        return list(self.weights) + list(self.biases)

    def weight_bytes(self):
        return sum(w.numel() * w.element_size() for w in self.weights)

    def row_major(self, i=0):
        """Weight i as a row-major [out, in] tensor (a copy if it is held shuffled; a gated pair keeps its interleaved rows)."""
        w = self.weights[i]
        return w.to_rows() if isinstance(w, ops.ShuffledWeight) else w

    def forward_glu(self, ctx, x, out, activation="silu", factor=1.0):
        """out [n, rows of one matrix] = factor * act(x @ gate.T + b) * (x @ up.T + b), in x's type (needs `gated`)."""
        return ops.linear_glu(x, self.weights[0], out, bias=self.biases[0] if self.biases else None,
                              activation=activation, factor=factor)

    def forward_act(self, ctx, x, out, activation):
        """out = act(x @ W.T (+ bias)) in x's type, the activation in the matrix kernel's epilogue; True if it ran
        (one packed matrix, more than 64 rows, K a multiple of 16 bytes), else nothing was written."""
        if len(self.weights) != 1 or self.gated or not ops.can_linear_act(x, self.weights[0]):
            return False
        w = self.weights[0]
        floats = ops.linear_workspace_bytes(w.dtype, x.shape[0], w.shape[0], w.shape[1]) // 4
        ws = ctx.workspace.get("linear.splitk.rows", (floats,), torch.float32) if floats else None
        ops.linear_act(x, w, out, activation, bias=self.biases[0] if self.biases else None, workspace=ws)
        return True

    def forward(self, ctx, x, out, residual=None):
        """out[:, columns] = x @ W.T (+ bias) (+ residual); out may be float32 or x's type."""
        if self.gated:
            raise RuntimeError("a gated pair of matrices has interleaved rows; use forward_glu")
        col = 0
        for i, w in enumerate(self.weights):
            rows = w.shape[0]
            target = out if len(self.weights) == 1 else out[:, col:col + rows]
            res = None
            if residual is not None:
                res = residual if len(self.weights) == 1 else residual[:, col:col + rows]
            ws = None
            if x.shape[0] <= 64:
                # Split-K scratch, sized once for the largest skinny batch so it never regrows.
                if i not in self._ws_floats:
                    self._ws_floats[i] = ops.linear_workspace_bytes(w.dtype, 64, rows, w.shape[1]) // 4
                if self._ws_floats[i]:
                    ws = ctx.workspace.get("linear.splitk", (self._ws_floats[i],), torch.float32)
            else:
                # few tiles for the chip (a few hundred rows, or large tiles against a matrix with few
                # columns and a long K): the tiled kernel splits K too
                # (a buffer of its own: growing with a prompt portion, it must not move the one captured decode steps hold)
                floats = ops.linear_workspace_bytes(w.dtype, x.shape[0], rows, w.shape[1]) // 4
                if floats:
                    ws = ctx.workspace.get("linear.splitk.rows", (floats,), torch.float32)
            ops.linear(x, w, target, bias=self.biases[i] if self.biases else None, residual=res, workspace=ws)
            col += rows
        return out

    # ---- leave the split-K sums to the next kernel -------------------------------------------
    def _partial_splits(self, n_rows, lda=None):
        """K ranges of `forward_partials` for N_ROWS rows, LDA elements apart (default: contiguous); 0: none.
        Up to 64 rows the streaming kernels' ranges depend on the matrix and on how many tiles of 16 rows
        there are; above, the tiled kernels choose them per row count and stride."""
        lda = self.weights[0].shape[1] if lda is None else int(lda)
        tile = (n_rows + 15) // 16 * 16 if n_rows <= 64 else n_rows       # up to 64 rows: the same for a tile of 16 rows
        key = ("splits", tile, lda)
        if key not in self._ws_floats:
            self._ws_floats[key] = ops.linear_partial_splits_rows(self.weights[0], tile, lda)
        return self._ws_floats[key]

    def deferrable(self, n_rows):
        """Can `forward_partials` run for N_ROWS rows, and is it worth it? (one packed matrix and a kernel
        that splits K for these rows anyway; a bias is NOT added to the partial sums: the caller's next
        kernel has to, or the caller must not defer)"""
        if len(self.weights) != 1 or n_rows < 1:
            return False
        return self._partial_splits(n_rows) > 0

    def forward_partials(self, ctx, x, tag):
        """float32 [splits, n, out] partial sums of x @ W.T (bias NOT added); see ops.linear_partials."""
        w = self.weights[0]
        n = x.shape[0]
        splits = self._partial_splits(n, x.stride(0) if n > 1 else None)
        if n <= 64:     # sized once for the largest such batch, so that it never regrows under a captured graph
            most = max(self._partial_splits(rows) for rows in (16, 32, 48, 64))
            buf = ctx.workspace.get("linear.partial." + tag, (most, 64, w.shape[0]), torch.float32)
        else:
            buf = ctx.workspace.get("linear.partial.rows." + tag, (splits, n, w.shape[0]), torch.float32)
        partial = buf.view(-1)[:splits * n * w.shape[0]].view(splits, n, w.shape[0])
        return ops.linear_partials(x, w, partial)


class JoinedLinear(Linear):
    """One product over several inputs laid side by side: out = [x_0 | x_1 | ...] @ [W_0 | W_1 | ...].T, the
    matrices W_i [out, in_i] joined along their columns into one weight, so that the outputs of parallel
    branches meet in one product (and one addition into the residual stream) instead of one each.

    pad_ins[i] = (unit, to) or None lays groups of input i out with tails of zeros, as `Linear(pad_in=)` does.
    """

    def __init__(self, names, in_features, out_features, pad_ins=None, suffix=".weight"):
        self.part_names = list(names)
        self.part_in = [int(k) for k in in_features]
        pads = list(pad_ins) if pad_ins else [None] * len(self.part_names)
        runs = [(k, *(pad if pad else (k, k))) for k, pad in zip(self.part_in, pads)]
        super().__init__(["|".join(self.part_names)], sum(self.part_in), [out_features], pad_in=runs,
                         suffixes=(suffix, ".bias"))
        self.part_runs = runs

    def tensor_specs(self):
        return [TensorSpec(name + self.suffixes[0], (self.out_features[0], k), MATRIX, NORMAL)
                for name, k in zip(self.part_names, self.part_in)]

    @property
    def device_in_parts(self):
        """Columns of each input on the device."""
        return [columns // unit * to for columns, unit, to in self.part_runs]

    def bind(self, tensors, dtype, device):
        joined = torch.cat([tensors.pop(name + self.suffixes[0]) for name in self.part_names], 1)
        super().bind({self.names[0] + self.suffixes[0]: joined}, dtype, device)

"""Mixers that run side by side on one input, and the two kinds of branch built here.

`ParallelMixer` reads h once: the input matrices of all its branches are one packed product, each branch
works on its own columns of the result, writes its output (times its weight in the sum, times the
block's residual multiplier) into its own columns of one buffer, and ONE joined output product adds
sum_b scale_b * W_o,b out_b into the residual stream.

`MixedHeadAttention`: grouped-query attention over the paged cache without rotation, whose scores lose
slope_h * distance, are mixed across heads by a learned [H, H] matrix before the softmax, see a sliding
window, and whose softmax has a learned sink per head; the values may have another size than the keys.

`GatedLinearRecurrence`: Griffin's recurrent block (De et al., "Griffin: Mixing Gated Linear Recurrences
with Local Attention for Efficient Language Models"): a gelu branch times the real-gated linear
recurrent unit of a short causal convolution of a linear branch; block-diagonal gates; the recurrence
and its gates in float32; state = the recurrence's S and the convolution's last inputs.
"""
from __future__ import annotations

import torch

from ..cache.spec import CacheNeed, FixedState, PagedKV
from ..kernels import ops
from ..weights.spec import IDENTITY_PLUS_NORMAL, MATRIX, NORMAL, VECTOR, TensorSpec
from .base import Mixer, Part
from .convolution import CausalConv
from .linear import JoinedLinear, Linear


def _round16(v):
    return (int(v) + 15) // 16 * 16


class MixerBranch(Part):
    """One of the mixers of a `ParallelMixer`.

    in_matrices():  [(checkpoint name, rows, has bias, (unit, to) padding of the rows or None), ...]
    out_matrix():   (checkpoint name, columns, (unit, to) padding of the columns or None)
    forward(ctx, run, proj, out, scale): proj holds this branch's columns of the packed input product,
    out its columns of the joined output product's input; writes scale * (the branch's result) there.
    """

    def in_matrices(self):
        raise NotImplementedError

    def out_matrix(self):
        raise NotImplementedError

    def cache_need(self):
        return None

    def forward(self, ctx, run, proj, out, scale):
        raise NotImplementedError


def distance_slopes(heads, base=8.0):
    """slope_h = 2^(-base (h + 1) / heads), h = 0 .. heads - 1."""
    return [2.0 ** (-base * (h + 1) / heads) for h in range(heads)]


class MixedHeadAttention(MixerBranch):
    def __init__(self, prefix, q_heads, kv_heads, key_dim, value_dim, scale, window=None, slope_base=8.0,
                 talk=True, sink=True, names=("q", "k", "v", "o", "talk", "sink")):
        if q_heads % kv_heads:
            raise ValueError("q_heads must be a multiple of kv_heads")
        if not (1 <= q_heads <= 32 and 1 <= key_dim <= 256 and 1 <= value_dim <= 256):
            raise ValueError("the mixed-head attention kernel takes up to 32 heads and sizes up to 256")
        self.prefix, self.names = prefix, tuple(names)
        self.q_heads, self.kv_heads = int(q_heads), int(kv_heads)
        self.key_dim, self.value_dim = int(key_dim), int(value_dim)
        # on the device a head is laid out in multiples of 16 elements, the tail zeros (exact: see GroupedQueryAttention)
        self.key_dev, self.value_dev = _round16(key_dim), _round16(value_dim)
        self.scale = float(scale)
        self.window = int(window) if window else None
        self.slope_base = slope_base
        self.has_talk, self.has_sink = bool(talk), bool(sink)
        self.talk = self.sink = self.slopes = None

    def _name(self, i):
        return self.prefix + self.names[i]

    def in_matrices(self):
        kd, vd = (self.key_dim, self.key_dev), (self.value_dim, self.value_dev)
        return [(self._name(0), self.q_heads * self.key_dim, False, kd),
                (self._name(1), self.kv_heads * self.key_dim, False, kd),
                (self._name(2), self.kv_heads * self.value_dim, False, vd)]

    def out_matrix(self):
        return (self._name(3), self.q_heads * self.value_dim, (self.value_dim, self.value_dev))

    def tensor_specs(self):
        specs = []
        if self.has_talk:
            specs.append(TensorSpec(self._name(4), (self.q_heads, self.q_heads), VECTOR, IDENTITY_PLUS_NORMAL))
        if self.has_sink:
            specs.append(TensorSpec(self._name(5), (self.q_heads,), VECTOR, NORMAL))
        return specs

    def bind(self, tensors, dtype, device):
        self.talk = tensors.pop(self._name(4)).contiguous() if self.has_talk else None
        self.sink = tensors.pop(self._name(5)).contiguous() if self.has_sink else None
        self.slopes = None
        if self.slope_base is not None:
            self.slopes = torch.tensor(distance_slopes(self.q_heads, self.slope_base), dtype=torch.float32, device=device)

    def weight_tensors(self):
        return [t for t in (self.talk, self.sink) if t is not None]

    def cache_need(self):
        return CacheNeed(paged=PagedKV(self.kv_heads, self.key_dev, self.window, self.value_dev))

    def forward(self, ctx, run, proj, out, scale):
        H, G, D, E = self.q_heads, self.kv_heads, self.key_dev, self.value_dev
        keys, values, g = ctx.cache.keys_values(run.cache_slot)
        values = values.view(values.shape[0], G, E, ctx.cache.page_size)
        group = ctx.groups[g]
        if run.writes_cache:
            ops.kv_store(proj, H * D, (H + G) * D, group.slot_mapping, keys, values, G, D, E)
        window = self.window or 0
        common = dict(window=window, talk=self.talk, sink=self.sink, slopes=self.slopes, out_scale=scale)
        if ctx.n_decode:
            longest = ctx.kv_bound if ctx.capturing else ctx.max_kv_len
            most = ctx.kv_capacity
            if window:
                longest, most = min(longest, window), min(most, window)
            splits = ops.attn_mixed_splits(ctx.n_decode, longest)
            ws = None
            if splits > 1:
                # sized for the most splits any length class can ask for, so that it never grows under a capture
                floats = ops.attn_mixed_workspace_floats(ctx.n_decode, 1, H, E, max(splits, ops.attn_mixed_splits(ctx.n_decode, most)))
                ws = ctx.workspace.get("attn.mixed.split", (floats,), torch.float32)
            ops.attn_mixed(proj, keys, values, group.block_table, ctx.q_start, ctx.kv_len, 0, ctx.n_decode, 1, out,
                           H, G, self.scale, splits=splits, workspace=ws, **common)
        if ctx.n_seqs > ctx.n_decode:
            n_seqs = ctx.n_seqs - ctx.n_decode
            longest = min(ctx.max_kv_len, window + ctx.max_q_len) if window else ctx.max_kv_len
            splits = ops.attn_mixed_prefill_splits(ctx.n_tokens - ctx.n_decode, n_seqs, longest)
            ws = None
            if splits > 1:
                floats = ops.attn_mixed_workspace_floats(n_seqs, ctx.max_q_len, H, E, splits)
                ws = ctx.workspace.get("attn.mixed.split.rows", (floats,), torch.float32)
            ops.attn_mixed(proj, keys, values, group.block_table, ctx.q_start, ctx.kv_len, ctx.n_decode,
                           n_seqs, ctx.max_q_len, out, H, G, self.scale, splits=splits, workspace=ws, **common)


class GatedLinearRecurrence(MixerBranch):
    def __init__(self, prefix, width, blocks, conv_taps, decay=8.0, state_prefix="recurrent",
                 names=("y", "x", "conv", "ra", "ri", "lam", "o"), bias_suffix=".b"):
        if width % blocks:
            raise ValueError("the recurrent width must be a multiple of its gate blocks")
        self.prefix, self.names, self.bias_suffix = prefix, tuple(names), bias_suffix
        self.width, self.blocks, self.decay = int(width), int(blocks), float(decay)
        self.width_dev = (self.width + 7) // 8 * 8          # rows of the packed product stay 16-byte aligned
        self.state_prefix = state_prefix
        self.conv = CausalConv(prefix + names[2], width, conv_taps, state_prefix + ".conv",
                               bias_name=prefix + names[2] + bias_suffix)
        self.gates = []
        self.lam = None

    def _name(self, i):
        return self.prefix + self.names[i]

    def parts(self):
        return [self.conv, *self.gates]

    def in_matrices(self):
        pad = (self.width, self.width_dev)
        return [(self._name(0), self.width, True, pad), (self._name(1), self.width, True, pad)]

    def out_matrix(self):
        return (self._name(6), self.width, (self.width, self.width_dev))

    def tensor_specs(self):
        B, n = self.blocks, self.width // self.blocks
        specs = self.conv.tensor_specs()
        for i in (3, 4):
            specs.append(TensorSpec(self._name(i), (B, n, n), MATRIX, NORMAL))
            specs.append(TensorSpec(self._name(i) + self.bias_suffix, (B, n), VECTOR, NORMAL))
        specs.append(TensorSpec(self._name(5), (self.width,), VECTOR, NORMAL))
        return specs

    def bind(self, tensors, dtype, device):
        self.conv.bind(tensors, dtype, device)
        n = self.width // self.blocks
        ra, ri = tensors.pop(self._name(3)), tensors.pop(self._name(4))
        ra_b, ri_b = tensors.pop(self._name(3) + self.bias_suffix), tensors.pop(self._name(4) + self.bias_suffix)
        self.gates = []
        # [blocks, 2n, n]: a block's recurrence gate rows, then its input gate rows; one kernel for all blocks
        # where the sizes allow it, else one product a block
        self.gate_weight = torch.cat([ra, ri], 1).contiguous()
        self.gate_bias = torch.cat([ra_b, ri_b], 1).contiguous().view(-1)
        probe = torch.empty(1, self.width_dev, dtype=self.gate_weight.dtype, device=self.gate_weight.device)[:, :self.width]
        self.gates_fused = torch.device(device).type == "cuda" and ops.can_block_diagonal(probe, self.gate_weight)
        for b in range(0 if not self.gates_fused else self.blocks, self.blocks):
            # the recurrence gate and the input gate of a block read the same inputs: one product for both
            name = f"{self.prefix}gates.{b}"
            gate = Linear([name], n, [2 * n], bias=True)
            gate.bind({name + ".weight": torch.cat([ra[b], ri[b]], 0), name + ".bias": torch.cat([ra_b[b], ri_b[b]], 0)},
                      dtype, device)
            self.gates.append(gate)
        self.lam = tensors.pop(self._name(5)).contiguous()

    def weight_tensors(self):
        return [self.lam] + ([self.gate_weight, self.gate_bias] if self.gates_fused else [])

    def cache_need(self):
        return CacheNeed(states=(self.conv.state_need(), (self.state_prefix + ".s", FixedState((self.width,), "float32"))))

    def forward(self, ctx, run, proj, out, scale):
        n, R = ctx.n_tokens, self.width
        branch, linear = proj[:, :R], proj[:, self.width_dev:self.width_dev + R]
        u = ctx.scratch("recurrent.u", (n, self.width_dev))[:, :R]                  # for the gates' products
        u32 = ctx.scratch("recurrent.u32", (n, R), torch.float32)                  # for the recurrence
        self.conv.forward(ctx, run, linear, out=u, out32=u32)
        gates = ctx.scratch("recurrent.gates", (n, 2 * R), torch.float32)
        bs = R // self.blocks
        if self.gates_fused:
            ops.block_diagonal(u, self.gate_weight, self.gate_bias, gates)
        for b, gate in enumerate(self.gates):
            gate.forward(ctx, u[:, b * bs:(b + 1) * bs], gates[:, 2 * b * bs:2 * (b + 1) * bs])
        state = ctx.cache.states[run.cache_slot][self.state_prefix + ".s"]
        longest = max(ctx.max_q_len, 1)
        ws = None
        floats = ops.gated_recurrence_workspace_floats(ctx.n_seqs, longest, R)
        if floats:
            ws = ctx.workspace.get("recurrent.chunks", (floats,), torch.float32)
        # (the columns beyond R meet zero columns of the output matrix, but must not hold NaN: the kernel clears them)
        ops.gated_recurrence(gates, u32, branch, self.lam, state, ctx.q_start, ctx.state_slots, ctx.n_seqs, longest,
                             out, self.blocks, self.decay, out_scale=scale, out_pad=self.width_dev - R, workspace=ws)


class ParallelMixer(Mixer):
    def __init__(self, hidden, branches, scales, out_scale=1.0, suffix=""):
        """branches: `MixerBranch`es reading the same input; scales: each one's weight in the sum;
        out_scale multiplies the whole sum (a block's residual multiplier)."""
        if len(branches) != len(scales) or not branches:
            raise ValueError("one scale per branch is needed")
        self.hidden, self.branches = int(hidden), list(branches)
        self.scales = [float(s) * float(out_scale) for s in scales]
        ins = [m for b in self.branches for m in b.in_matrices()]
        self.proj = Linear([m[0] for m in ins], hidden, [m[1] for m in ins], bias=[m[2] for m in ins],
                           pad_out=[m[3] for m in ins], suffixes=(suffix, ".b"))
        outs = [b.out_matrix() for b in self.branches]
        self.out = JoinedLinear([o[0] for o in outs], [o[1] for o in outs], hidden, pad_ins=[o[2] for o in outs],
                                suffix=suffix)
        widths, at = self.proj.device_out, 0
        self.in_columns = []
        for b in self.branches:
            k = len(b.in_matrices())
            self.in_columns.append((sum(widths[:at]), sum(widths[at:at + k])))
            at += k
        self.out_columns, col = [], 0
        for w in self.out.device_in_parts:
            self.out_columns.append((col, w))
            col += w

    def parts(self):
        return [self.proj, self.out, *self.branches]

    def tensor_specs(self):
        return self.proj.tensor_specs() + self.out.tensor_specs() + [s for b in self.branches for s in b.tensor_specs()]

    def bind(self, tensors, dtype, device):
        self.proj.bind(tensors, dtype, device)
        self.out.bind(tensors, dtype, device)
        for b in self.branches:
            b.bind(tensors, dtype, device)

    def cache_need(self):
        need = CacheNeed()
        for b in self.branches:
            need = need.merged(b.cache_need())
        return need

    def forward(self, ctx, run, h, x):
        n = ctx.n_tokens
        proj = ctx.scratch("parallel.proj", (n, sum(self.proj.device_out)))
        self.proj.forward(ctx, h, proj)
        joined = ctx.scratch("parallel.out", (n, self.out.device_in))
        for b, (c0, w), (o0, ow), scale in zip(self.branches, self.in_columns, self.out_columns, self.scales):
            b.forward(ctx, run, proj[:, c0:c0 + w], joined[:, o0:o0 + ow], scale)
        self.out.forward(ctx, joined, x, residual=x)
        return None

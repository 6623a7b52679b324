"""Attention over a cached latent.

Every token leaves ONE normed vector c (L elements) and one rotated key part kr (R elements) that all heads share;
head a's key is [W_uk,a c | kr], its value W_uv,a c, its query [D unrotated | R rotated] elements:

    score_a(i, j) = scale * (q_plain,a(i) . W_uk,a c_j + q_turned,a(i) . kr_j),   causal softmax,   out = W_o [.. W_uv,a sum_j p c_j ..]

Only c and kr are cached. The products with W_uk and W_uv are moved to the query side and the output side (one
small matrix per head each, `ops.head_linear`), so that the attention itself runs over one key/value head whose
key row is [c | kr] and whose value is c, for all query heads at once; the engine's paged cache holds it like any
other group (one key/value head, values of another size than keys). A layer may read the cache slot of another
layer (`LayerRun(writes_cache=False)`): it then has no down-projection of its own (`own_latent=False`) and uses that
layer's c and kr with its own queries and its own W_uk, W_uv.
"""
from __future__ import annotations

import torch

from ..cache.spec import CacheNeed, PagedKV
from ..kernels import ops
from ..weights.spec import MATRIX, NORMAL, ONE_PLUS_NORMAL, VECTOR, TensorSpec
from .base import Mixer
from .linear import Linear, pad_groups


def _round_up(v, m):
    return (int(v) + m - 1) // m * m


class LatentAttention(Mixer):
    def __init__(self, prefix, hidden, heads, dim, rot_dim, value_dim, latent, scale, position, eps, own_latent=True,
                 names=("q", "dkv", "dkv.norm", "uk", "uv", "o")):
        """position: a rotary encoding over `rot_dim` elements (its `rotary_dim` may be smaller: the rest of the
        rotated part passes unchanged). scale multiplies the scores as given."""
        self.prefix, self.names = prefix, tuple(names)
        self.hidden, self.heads = int(hidden), int(heads)
        self.dim, self.rot_dim, self.value_dim, self.latent = int(dim), int(rot_dim), int(value_dim), int(latent)
        if min(self.heads, self.dim, self.rot_dim, self.value_dim, self.latent) <= 0:
            raise ValueError("heads and sizes must be positive")
        if position.rotary_dim <= 0 or position.rotary_dim > self.rot_dim or position.pairing != "half":
            raise ValueError("the rotated part needs a rotary encoding of at most rot_dim elements with the 'half' pairing")
        # sizes on the device: tails of zeros, which add nothing to a product
        self.dim_dev, self.value_dev = _round_up(dim, 8), _round_up(value_dim, 8)
        self.latent_dev, self.rot_dev = _round_up(latent, 16), _round_up(rot_dim, 16)
        self.key_dev = self.latent_dev + self.rot_dev
        if self.heads > 32 or self.key_dev > 256:
            raise ValueError("the attention kernel takes up to 32 heads and latent + rotated sizes up to 256")
        self.scale, self.eps, self.position, self.own_latent = float(scale), float(eps), position, bool(own_latent)
        self.proj = self.absorb = self.expand = self.latent_norm = None
        self.o = Linear([prefix + self.names[5]], heads * value_dim, [hidden], pad_in=(self.value_dim, self.value_dev),
                        suffixes=("", ".bias"))

    def _name(self, i):
        return self.prefix + self.names[i]

    def parts(self):
        return [p for p in (self.proj, self.o, self.position) if p is not None]

    def tensor_specs(self):
        H, D, R, E, L, C = self.heads, self.dim, self.rot_dim, self.value_dim, self.latent, self.hidden
        specs = [TensorSpec(self._name(0), (H * (D + R), C), MATRIX, NORMAL)]
        if self.own_latent:
            specs += [TensorSpec(self._name(1), (L + R, C), MATRIX, NORMAL),
                      TensorSpec(self._name(2), (L,), VECTOR, ONE_PLUS_NORMAL)]
        specs += [TensorSpec(self._name(3), (H * D, L), MATRIX, NORMAL), TensorSpec(self._name(4), (H * E, L), MATRIX, NORMAL)]
        return specs + self.o.tensor_specs()

    def bind(self, tensors, dtype, device):
        H, D, R, E, L = self.heads, self.dim, self.rot_dim, self.value_dim, self.latent
        Dp, Rp, Ep, Lp = self.dim_dev, self.rot_dev, self.value_dev, self.latent_dev
        q = tensors.pop(self._name(0)).view(H, D + R, self.hidden)
        # one packed product: [all heads' unrotated query parts | all heads' rotated parts | latent | shared key part]
        rows = [pad_groups(q[:, :D].reshape(H * D, -1), 0, D, Dp), pad_groups(q[:, D:].reshape(H * R, -1), 0, R, Rp)]
        if self.own_latent:
            down = tensors.pop(self._name(1))
            rows += [pad_groups(down[:L], 0, L, Lp), pad_groups(down[L:], 0, R, Rp)]
            self.latent_norm = tensors.pop(self._name(2)).contiguous()
        packed = torch.cat(rows, 0).contiguous()
        self.q_col, self.c_col, self.kr_col = H * Dp, H * (Dp + Rp), H * (Dp + Rp) + Lp
        self.proj_width = packed.shape[0]
        name = self.prefix + "packed"
        self.proj = Linear([name], self.hidden, [self.proj_width])
        self.proj.bind({name + ".weight": packed}, dtype, device)
        del q, rows, packed
        # query side: q_latent,a = W_uk,a^T q_plain,a ([Lp, Dp] per head); output side: W_uv,a ([Ep, Lp] per head)
        uk = tensors.pop(self._name(3)).view(H, D, L)
        self.absorb = uk.new_zeros(H, Lp, Dp)
        self.absorb[:, :L, :D] = uk.transpose(1, 2)
        uv = tensors.pop(self._name(4)).view(H, E, L)
        self.expand = uv.new_zeros(H, Ep, Lp)
        self.expand[:, :E, :L] = uv
        self.o.bind(tensors, dtype, device)
        self.position.bind(tensors, dtype, device)

    def weight_tensors(self):
        return [t for t in (self.absorb, self.expand, self.latent_norm) if t is not None]

    def cache_need(self):
        return CacheNeed(paged=PagedKV(1, self.key_dev, None, self.latent_dev))

    def forward(self, ctx, run, h, x, accumulate=True):
        if run.writes_cache != self.own_latent:
            raise RuntimeError("a layer with a latent of its own writes its cache slot; one without reads another layer's")
        n, H = ctx.n_tokens, self.heads
        Lp, Rp, K = self.latent_dev, self.rot_dev, self.key_dev
        proj = ctx.scratch("latent.proj", (n, self.proj_width))
        self.proj.forward(ctx, h, proj)
        cos, sin = self.position.tables(ctx)
        keys, values, g = ctx.cache.keys_values(run.cache_slot)
        values = values.view(values.shape[0], 1, Lp, ctx.cache.page_size)
        group = ctx.groups[g]
        q = ctx.scratch("latent.q", (n, H * K))
        store = dict(keys=keys, values=values, slots=group.slot_mapping) if self.own_latent else {}
        ops.latent_finish(proj, self.q_col, self.c_col, self.kr_col, cos, sin, self.latent_norm, q, H, self.latent, Lp, Rp,
                          self.eps, **store)
        ops.head_linear(proj, self.dim_dev, self.absorb, q, K)
        mixed = ctx.scratch("latent.mixed", (n, H * Lp))
        if ctx.n_decode:
            longest = ctx.kv_bound if ctx.capturing else ctx.max_kv_len
            splits = ops.attn_mixed_splits(ctx.n_decode, longest)
            ws = None
            if splits > 1:
                # sized for the most splits any length class can ask for, so that it never grows under a capture
                floats = ops.attn_mixed_workspace_floats(ctx.n_decode, 1, H, Lp,
                                                         max(splits, ops.attn_mixed_splits(ctx.n_decode, ctx.kv_capacity)))
                ws = ctx.workspace.get("attn.mixed.split", (floats,), torch.float32)
            ops.attn_mixed(q, keys, values, group.block_table, ctx.q_start, ctx.kv_len, 0, ctx.n_decode, 1, mixed, H, 1,
                           self.scale, splits=splits, workspace=ws)
        if ctx.n_seqs > ctx.n_decode:
            n_seqs = ctx.n_seqs - ctx.n_decode
            splits = ops.attn_mixed_prefill_splits(ctx.n_tokens - ctx.n_decode, n_seqs, ctx.max_kv_len)
            ws = None
            if splits > 1:
                floats = ops.attn_mixed_workspace_floats(n_seqs, ctx.max_q_len, H, Lp, splits)
                ws = ctx.workspace.get("attn.mixed.split.rows", (floats,), torch.float32)
            ops.attn_mixed(q, keys, values, group.block_table, ctx.q_start, ctx.kv_len, ctx.n_decode, n_seqs, ctx.max_q_len,
                           mixed, H, 1, self.scale, splits=splits, workspace=ws)
        out = ctx.scratch("latent.out", (n, H * self.value_dev))
        ops.head_linear(mixed, Lp, self.expand, out, self.value_dev)
        if ctx.defer_sums and self.o.deferrable(n):
            return self.o.forward_partials(ctx, out, "o")          # whoever norms next adds them up
        self.o.forward(ctx, out, x, residual=x if accumulate else None)
        return None

"""A plain, slow implementation of the Dinutar decoder, one function per mechanism.

Written from the design's equations with ordinary tensor operations on whole sequences; it shares no
code with the package and keeps no cache: a sequence is always computed from its first token. The
tests compare the engine with it (prefill, decoding, portions and batches all have to give what this
gives for the whole sequence).

Notation: T tokens, C the model's width, H heads, D the unrotated query/key size of a head, R its
rotated size, E the value size, L the latent size, V the vocabulary.
"""
from __future__ import annotations

import math

import torch


def rms_unit(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def rms_norm(x, weight, eps):
    return rms_unit(x, eps) * weight


def bigram_rows(tokens, buckets, mul_prev, mul_cur):
    """Row of the bigram table for every token: a hash of (previous token, token); the first token of a
    sequence, which has no previous one, takes the table's last row (number `buckets`)."""
    rows = [buckets]
    for prev, cur in zip(tokens[:-1], tokens[1:]):
        rows.append((prev * mul_prev + cur * mul_cur) % buckets)
    return rows


def embed(tokens, table, bigram, scale, buckets, mul_prev, mul_cur, norm_weight, eps):
    ids = [int(t) for t in tokens]
    rows = torch.tensor(bigram_rows(ids, buckets, mul_prev, mul_cur), dtype=torch.long)
    x = table[torch.tensor(ids, dtype=torch.long)] * scale + bigram[rows]
    return rms_norm(x, norm_weight, eps)


def rotary_frequencies(dims, base, scaling=None, dtype=torch.float64):
    """(frequencies [dims / 2], factor on cos and sin). With `scaling` (factor, original, fast, slow): the
    frequencies whose wavelength is long against the original context are divided by the factor, those
    that turn fast are kept, a linear ramp over the pair index lies between, and cos and sin grow by
    0.1 ln(factor) + 1."""
    half = dims // 2
    i = torch.arange(half, dtype=dtype)
    f = base ** (-2.0 * i / dims)
    if not scaling:
        return f, 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])

    def pair_of(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(pair_of(float(scaling["fast"]))), 0)
    hi = min(math.ceil(pair_of(float(scaling["slow"]))), dims - 1)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate(x, positions, dims, base, scaling=None):
    """x [T, heads, >= dims]: the first `dims` elements of every head turn, element i with i + dims / 2."""
    f, mag = rotary_frequencies(dims, base, scaling, x.dtype)
    angle = positions.to(x.dtype).view(-1, 1, 1) * f.view(1, 1, -1)
    cos, sin = torch.cos(angle) * mag, torch.sin(angle) * mag
    half = dims // 2
    u, v, rest = x[..., :half], x[..., half:dims], x[..., dims:]
    return torch.cat([u * cos - v * sin, v * cos + u * sin, rest], -1)


def latent_from(h, w_dkv, latent_norm, L, eps, positions, rot):
    """What a latent-attention layer caches for its tokens: the normed latent [T, L] and the one rotated
    key part [T, R] that all heads share."""
    down = h @ w_dkv.T
    latent = rms_norm(down[:, :L], latent_norm, eps)
    shared = rotate(down[:, L:].unsqueeze(1), positions, rot["dims"], rot["base"], rot.get("scaling"))[:, 0]
    return latent, shared


def latent_attention(h, latent, shared, w_q, w_uk, w_uv, w_o, H, D, R, E, scale, positions, rot):
    """Causal softmax attention whose keys and values are expanded from the latent: key of head a =
    [W_uk,a latent | shared], value = W_uv,a latent; a query head is [D unrotated | R rotated]."""
    T = h.shape[0]
    q = (h @ w_q.T).view(T, H, D + R)
    q_plain = q[..., :D]
    q_turn = rotate(q[..., D:], positions, rot["dims"], rot["base"], rot.get("scaling"))
    k_plain = (latent @ w_uk.T).view(T, H, D)
    value = (latent @ w_uv.T).view(T, H, E)
    s = (torch.einsum("iad,jad->aij", q_plain, k_plain) + torch.einsum("iar,jr->aij", q_turn, shared)) * scale
    i = torch.arange(T).view(T, 1)
    j = torch.arange(T).view(1, T)
    s = s.masked_fill(j > i, float("-inf"))
    p = torch.softmax(s, -1)
    o = torch.einsum("aij,jae->iae", p, value).reshape(T, H * E)
    return o @ w_o.T


def retention(h, w_q, w_k, w_v, w_g, w_o, H, D, E, decay, eps, positions, rot):
    """Linear attention with a fixed decay per head, token by token: S <- decay S + k v^T, o = S^T q;
    each head's o over its root mean square, times silu of a gate, then the output matrix."""
    T = h.shape[0]
    q, k = (h @ w_q.T).view(T, H, D), (h @ w_k.T).view(T, H, D)
    if rot is not None:
        q = rotate(q, positions, rot["dims"], rot["base"], rot.get("scaling"))
        k = rotate(k, positions, rot["dims"], rot["base"], rot.get("scaling"))
    k = k * D ** -0.5
    v = (h @ w_v.T).view(T, H, E)
    g = h @ w_g.T
    state = h.new_zeros(H, D, E)
    gamma = torch.tensor(decay, dtype=h.dtype).view(H, 1, 1)
    out = []
    for t in range(T):
        state = gamma * state + k[t].unsqueeze(-1) * v[t].unsqueeze(-2)
        out.append(torch.einsum("ade,ad->ae", state, q[t]))
    o = rms_unit(torch.stack(out), eps).reshape(T, H * E)
    return (o * torch.nn.functional.silu(g)) @ w_o.T


def relu_squared_ff(h, w_up, w_down):
    return torch.relu(h @ w_up.T) ** 2 @ w_down.T


def forward(config, weights, tokens, dtype=torch.float64, layers_out=None):
    """Logits [T, V] of the whole sequence TOKENS. config: config.json's dictionary; weights: name -> tensor.
    layers_out: a list that receives the residual stream after every layer."""
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
    eps, alpha = config["norm"]["eps"], config["postln_alpha"]
    e = config["embedding"]
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    positions = torch.arange(tokens.numel())
    x = embed(tokens, w["embed"], w["bigram"], e["scale"], e["bigram"]["buckets"], e["bigram"]["mul_prev"],
              e["bigram"]["mul_cur"], w["embed.norm"], eps)
    cached = {}
    for n, layer in enumerate(config["layers"]):
        p, m = f"l{n}.", layer["mixer"]
        if layer["type"] == "latent_attention":
            source = m.get("kv_from")
            if source is None:
                cached[n] = latent_from(x, w[p + "mix.dkv"], w[p + "mix.dkv.norm"], m["kv_rank"], eps, positions, m["rot"])
                source = n
            latent, shared = cached[source]
            y = latent_attention(x, latent, shared, w[p + "mix.q"], w[p + "mix.uk"], w[p + "mix.uv"], w[p + "mix.o"],
                                 m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["scale"], positions, m["rot"])
        elif layer["type"] == "retention":
            y = retention(x, w[p + "mix.q"], w[p + "mix.k"], w[p + "mix.v"], w[p + "mix.g"], w[p + "mix.o"],
                          m["heads"], m["dim"], m["vdim"], m["decay"], eps, positions, m.get("rot"))
        else:
            raise ValueError(layer["type"])
        x = rms_norm(alpha * x + w[p + "ls1"] * y, w[p + "norm1"], eps)
        if layer.get("mlp"):
            y = relu_squared_ff(x, w[p + "mlp.up"], w[p + "mlp.down"])
            x = rms_norm(alpha * x + w[p + "ls2"] * y, w[p + "norm2"], eps)
        if layers_out is not None:
            layers_out.append(x)
    x = rms_norm(x, w["final.norm"], eps)
    return x @ w["embed"].T

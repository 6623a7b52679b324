"""A plain, slow implementation of the Kanavik decoder, one function per mechanism.

Written from the design's equations with ordinary tensor operations on whole sequences; it shares no
code with the package and keeps no cache: a sequence is always computed from its first token. The
tests compare the engine with it (prefill, decoding, portions, batches all have to give what this
gives for the whole sequence).

Notation: T tokens, C the model's width, H query heads, G key/value heads, D the query/key size,
E the value size, W the window, R the recurrent width, K taps of a causal convolution.
"""
from __future__ import annotations

import math

import torch


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def rms_unit(x, eps):
    """x over the root of (its mean square + eps), per row."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def rms_norm(x, weight, eps):
    return rms_unit(x, eps) * weight


def causal_conv(h, taps_weight):
    """[T, C] -> [T, C]: out_t = sum_j w[:, j] h_(t - K + 1 + j); the last column meets the current token,
    rows before the sequence count as zeros."""
    T, C = h.shape
    K = taps_weight.shape[1]
    padded = torch.cat([h.new_zeros(K - 1, C), h], 0)
    out = h.new_zeros(T, C)
    for j in range(K):
        out = out + padded[j:j + T] * taps_weight[:, j]
    return out


def input_conv(h, taps_weight):
    """What a sublayer reads instead of h: h plus its causal convolution."""
    return h + causal_conv(h, taps_weight)


def distance_slopes(H, dtype=torch.float64):
    return torch.tensor([2.0 ** (-8.0 * (h + 1) / H) for h in range(H)], dtype=dtype)


def mixed_head_attention(q, k, v, scale, window, talk, sink):
    """q [T, H, D], k [T, G, D], v [T, G, E] -> [T, H, E].

    score_h(i, j) = scale q_ih . k_jg - slope_h (i - j); scores are mixed over heads with `talk`
    [H, H]; position i sees 0 <= i - j < window; the softmax's denominator holds exp(sink_h) once more.
    """
    T, H, D = q.shape
    G = k.shape[1]
    rep = H // G
    kk = k.repeat_interleave(rep, 1)                   # head h reads key/value head h // rep
    vv = v.repeat_interleave(rep, 1)
    s = torch.einsum("ihd,jhd->hij", q, kk) * scale
    i = torch.arange(T).view(T, 1)
    j = torch.arange(T).view(1, T)
    dist = (i - j).to(s.dtype)
    s = s - distance_slopes(H, s.dtype).view(H, 1, 1) * dist
    s = torch.einsum("hg,gij->hij", talk, s)
    seen = (i - j >= 0) & (i - j < window)
    s = s.masked_fill(~seen, float("-inf"))
    top = torch.maximum(s.max(-1, keepdim=True).values, sink.view(H, 1, 1))
    e = torch.exp(s - top)
    denom = e.sum(-1, keepdim=True) + torch.exp(sink.view(H, 1, 1) - top)
    p = e / denom
    return torch.einsum("hij,jhe->ihe", p, vv)


def gated_recurrence(u, gate_a, gate_i, lam, state=None):
    """The real-gated linear recurrent unit over [T, R]: a = exp(-8 r softplus(lam)),
    S_t = a S_(t-1) + sqrt(1 - a^2) i u, from S = 0. Returns every S_t."""
    T, R = u.shape
    S = u.new_zeros(R) if state is None else state
    decay_unit = torch.nn.functional.softplus(lam)
    out = []
    for t in range(T):
        a = torch.exp(-8.0 * gate_a[t] * decay_unit)
        S = a * S + torch.sqrt(1.0 - a * a) * gate_i[t] * u[t]
        out.append(S)
    return torch.stack(out)


def block_diagonal(u, weight, bias):
    """u [T, R] in `blocks` equal parts, part b times weight[b] ([out, in]) plus bias[b]."""
    B, n_out, n_in = weight.shape
    parts = u.view(u.shape[0], B, n_in)
    return (torch.einsum("tbi,boi->tbo", parts, weight) + bias).reshape(u.shape[0], B * n_out)


def recurrent_branch(h, w, p):
    """Griffin's recurrent block: gelu branch times the recurrence of the convolved linear branch."""
    y = gelu_tanh(h @ w[p + "y"].T + w[p + "y.b"])
    u = causal_conv(h @ w[p + "x"].T + w[p + "x.b"], w[p + "conv"]) + w[p + "conv.b"]
    r = torch.sigmoid(block_diagonal(u, w[p + "ra"], w[p + "ra.b"]))
    i = torch.sigmoid(block_diagonal(u, w[p + "ri"], w[p + "ri.b"]))
    S = gated_recurrence(u, r, i, w[p + "lam"])
    return (S * y) @ w[p + "o"].T


def attention_branch(h, w, p, spec):
    T = h.shape[0]
    H, G, D, E = spec["heads"], spec["kv_heads"], spec["dim"], spec["vdim"]
    q = (h @ w[p + "q"].T).view(T, H, D)
    k = (h @ w[p + "k"].T).view(T, G, D)
    v = (h @ w[p + "v"].T).view(T, G, E)
    window = spec["mask"]["size"] if spec.get("mask") else T + 1          # no mask entry: every earlier key is seen
    o = mixed_head_attention(q, k, v, spec["scale"], window, w[p + "talk"], w[p + "sink"])
    return o.reshape(T, H * E) @ w[p + "o"].T


def parallel_mixer(h, w, p, spec):
    left = attention_branch(h, w, p + "left.", spec["left"])
    right = recurrent_branch(h, w, p + "right.")
    return spec["left_scale"] * left + spec["right_scale"] * right


def dense_feed_forward(h, w, p):
    return (gelu_tanh(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def token_side_input(x, tokens, w, layer, side_dim, eps):
    """The per-layer token input: y = proj(gelu(gate x) * e), returned divided by its root mean square
    and scaled by the plain weight `side.norm`."""
    e = w["side.embed"][tokens][:, layer * side_dim:(layer + 1) * side_dim]
    g = gelu_tanh(x @ w[f"l{layer}.side.gate"].T) * e
    y = g @ w[f"l{layer}.side.proj"].T
    return rms_unit(y, eps) * w[f"l{layer}.side.norm"]


def forward(config, weights, tokens, dtype=torch.float64, layers_out=None):
    """Logits [T, vocab] of a whole sequence. `layers_out`, a list, receives every layer's result
    (before the depth average)."""
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    T = tokens.shape[0]
    eps = config["norm"]["eps"]
    m = config["residual_mult"]
    x = w["embed"][tokens] + w["pos"][:T]
    results = [x]
    for i, layer in enumerate(config["layers"]):
        p = f"l{i}."
        if layer["type"] != "parallel":
            raise ValueError(layer["type"])
        h = input_conv(rms_norm(x, w[p + "norm1"], eps), w[p + "canon1"])
        x = x + m * parallel_mixer(h, w, p + "mix.", layer["mixer"])
        if layer.get("mlp"):
            h = input_conv(rms_norm(x, w[p + "norm2"], eps), w[p + "canon2"])
            x = x + m * dense_feed_forward(h, w, p + "mlp.")
        if config.get("token_side"):
            x = x + m * token_side_input(x, tokens, w, i, config["token_side"]["dim"], eps)
        results.append(x)
        if layers_out is not None:
            layers_out.append(x)
        x = sum(w[p + "dwa"][j] * results[j] for j in range(i + 2))
    return rms_norm(x, w["final.norm"], eps) @ w["head"].T

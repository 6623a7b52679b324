"""Small Kanavik configurations, weights made for testing, and a driver of the package's step function.

The configurations differ from each other in every size, in the order and the sizes of their layers,
and in what the design allows to be absent (a layer without a feed-forward, a model without the
per-layer token input, a layer without a window). Weights are drawn so that every path matters: the
head-mixing matrix is far from the identity, sinks and decays are of order one, the depth mix has no
small entries.
"""
from __future__ import annotations

import json
import math
from pathlib import Path

import numpy as np
import torch


def layer(heads, kv_heads, dim, vdim, window, scale, rwidth, blocks, conv, ff, left_scale=0.9, right_scale=1.3):
    left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if window:
        left["mask"] = {"size": window}
    return {"type": "parallel",
            "mixer": {"left": left, "right": {"width": rwidth, "blocks": blocks, "conv": conv},
                      "left_scale": left_scale, "right_scale": right_scale},
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


def config(layers, width, vocab, taps, side, mult=0.6, eps=1e-5, max_positions=640):
    c = {"architecture": "Kanavik", "vocab": vocab, "width": width, "max_positions": max_positions,
         "norm": {"eps": eps}, "residual_mult": mult, "canon": {"taps": taps}, "layers": layers}
    if side:
        c["token_side"] = {"dim": side}
    return c


# sizes that are no multiples of 16 (heads, values, recurrent width, side input), one key/value head per query
# head, a window of 7, taps 4 and 2, a layer without a feed-forward, a window longer than any test sequence
CONFIG_ODD = config([layer(4, 4, 24, 40, 7, 0.2, 36, 3, 4, 136),
                     layer(6, 2, 32, 16, 33, 0.15, 64, 1, 2, None, 1.1, 0.4),
                     layer(1, 1, 80, 96, 1000, 0.1, 24, 2, 1, 64, 0.5, 1.0)],
                    width=96, vocab=211, taps=4, side=12)
# all heads on one key/value head, a window of one page and one of 1, no per-layer token input, no window at all in one layer
CONFIG_WIDE = config([layer(12, 1, 16, 16, 16, 0.25, 128, 4, 3, 192),
                      layer(2, 1, 64, 128, 1, 0.12, 48, 2, 5, 200),
                      layer(8, 4, 48, 48, None, 0.14, 32, 32, 2, 96)],
                     width=128, vocab=300, taps=2, side=0, mult=1.0)
# one layer, taps of 1 (no state at all in the input convolutions)
CONFIG_ONE = config([layer(2, 2, 16, 32, 20, 0.25, 16, 1, 2, 48)], width=48, vocab=97, taps=1, side=8)

CONFIGS = {"odd": CONFIG_ODD, "wide": CONFIG_WIDE, "one": CONFIG_ONE}


def tensor_shapes(c):
    C, L = c["width"], len(c["layers"])
    shapes = {"embed": (c["vocab"], C), "pos": (c["max_positions"], C), "final.norm": (C,), "head": (c["vocab"], C)}
    side = (c.get("token_side") or {}).get("dim", 0)
    if side:
        shapes["side.embed"] = (c["vocab"], L * side)
    taps = c["canon"]["taps"]
    for i, lay in enumerate(c["layers"]):
        p = f"l{i}."
        left, right = lay["mixer"]["left"], lay["mixer"]["right"]
        H, G, D, E, R, B = left["heads"], left["kv_heads"], left["dim"], left["vdim"], right["width"], right["blocks"]
        shapes.update({p + "norm1": (C,), p + "canon1": (C, taps), p + "dwa": (i + 2,),
                       p + "mix.left.q": (H * D, C), p + "mix.left.k": (G * D, C), p + "mix.left.v": (G * E, C),
                       p + "mix.left.talk": (H, H), p + "mix.left.sink": (H,), p + "mix.left.o": (C, H * E),
                       p + "mix.right.y": (R, C), p + "mix.right.y.b": (R,), p + "mix.right.x": (R, C),
                       p + "mix.right.x.b": (R,), p + "mix.right.conv": (R, right["conv"]), p + "mix.right.conv.b": (R,),
                       p + "mix.right.ra": (B, R // B, R // B), p + "mix.right.ra.b": (B, R // B),
                       p + "mix.right.ri": (B, R // B, R // B), p + "mix.right.ri.b": (B, R // B),
                       p + "mix.right.lam": (R,), p + "mix.right.o": (C, R)})
        if lay["mlp"]:
            F = lay["mlp"]["ff"]
            shapes.update({p + "norm2": (C,), p + "canon2": (C, taps), p + "mlp.gate": (F, C), p + "mlp.up": (F, C),
                           p + "mlp.down": (C, F)})
        if side:
            shapes.update({p + "side.gate": (side, C), p + "side.proj": (C, side), p + "side.norm": (C,)})
    return shapes


def make_weights(c, seed):
    """{name: bfloat16 tensor}: what a checkpoint of configuration C holds."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(c).items():
        leaf = name.split(".")[-1]
        normal = torch.randn(shape, generator=g)
        if name in ("embed", "side.embed"):
            t = normal
        elif name == "pos":
            t = 0.5 * normal
        elif leaf in ("norm1", "norm2", "norm") or name == "final.norm":
            t = 1.0 + 0.2 * normal
        elif leaf == "talk":
            t = torch.eye(shape[0]) + 0.4 * normal
        elif leaf in ("sink", "lam"):
            t = normal
        elif leaf == "dwa":
            t = (0.4 + torch.rand(shape, generator=g)) / math.sqrt(shape[0])
        elif leaf in ("canon1", "canon2", "conv"):
            t = 0.5 * normal
        elif leaf == "b":
            t = 0.3 * normal
        else:                                             # linear maps [out, in] (the last size is the input's)
            t = normal / math.sqrt(shape[-1])
        out[name] = t.to(torch.bfloat16)
    return out


def write_folder(folder, c, weights):
    from safetensors.torch import save_file
    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    (folder / "config.json").write_text(json.dumps(c, indent=1))
    save_file({k: v.contiguous() for k, v in weights.items()}, str(folder / "model.safetensors"))
    return folder


def row_error(got, want):
    """Per row: root mean square of the difference (its mean taken off) over the root mean square of WANT."""
    d = np.asarray(got, dtype=np.float64) - np.asarray(want, dtype=np.float64)
    d = d - d.mean(-1, keepdims=True)
    w = np.asarray(want, dtype=np.float64)
    scale = np.sqrt(((w - w.mean(-1, keepdims=True)) ** 2).mean())
    return np.sqrt((d ** 2).mean(-1)) / scale


class Driver:
    """The package's loader, cache manager and step function around a model folder."""

    def __init__(self, folder, dtype, pages=64, page_size=16, max_requests=4, graphs=True, max_step_tokens=64):
        from tessweave_engine_amd.cache import CacheManager
        from tessweave_engine_amd.engine.step import Stepper
        from tessweave_engine_amd.weights import load_model
        self.model = load_model(folder, dtype=dtype, device="cuda:0")
        self.cache = CacheManager(self.model.cache_layout(), page_size, pages, max_requests, dtype=dtype,
                                  device=self.model.device, prefix_cache=False, max_request_tokens=pages * page_size)
        self.stepper = Stepper(self.model, self.cache, max_step_tokens=max_step_tokens, use_graphs=graphs)
        self.live = {}
        self.at = {}

    def step(self, parts, tokens_of):
        """PARTS: [(request id, count)]; runs each request's next COUNT tokens as one batch and returns
        {request id: (first position, logits [count, vocab])}."""
        from tessweave_engine_amd.engine.step import StepEntry
        entries, spans = [], []
        for rid, count in parts:
            if rid not in self.live:
                self.live[rid] = self.cache.open(rid)
                self.at[rid] = 0
            lo = self.at[rid]
            entries.append(StepEntry(self.live[rid], list(tokens_of[rid][lo:lo + count]), list(range(count))))
            spans.append((rid, lo, count))
            self.at[rid] = lo + count
        logits = self.stepper.step(entries).cpu().numpy()
        out, row = {}, 0
        for rid, lo, count in spans:
            out[rid] = (lo, logits[row:row + count].copy())
            row += count
        return out

    def end(self, rid):
        self.cache.close(self.live.pop(rid))
        self.cache.check()

    def run(self, schedule, tokens_of):
        """All steps of SCHEDULE; a request ends when its tokens are used up. Returns {id: logits [T, vocab]}."""
        got = {rid: np.zeros((len(toks), self.model.vocab_size), dtype=np.float32) for rid, toks in tokens_of.items()}
        for parts in schedule:
            for rid, (lo, rows) in self.step(parts, tokens_of).items():
                got[rid][lo:lo + len(rows)] = rows
                if self.at[rid] == len(tokens_of[rid]):
                    self.end(rid)
        return got

    def close(self):
        self.stepper.close()

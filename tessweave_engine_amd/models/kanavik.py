"""The Kanavik decoder: its typed configuration and its model assembled from parts.

config.json gives every size and every constant that differs between models of the design:

    architecture "Kanavik", vocab, width, max_positions, norm.eps, residual_mult, canon.taps, token_side.dim,
    layers: [{type: "parallel", mixer: {left: {heads, kv_heads, dim, vdim, scale, mask.size}, right: {width,
              blocks, conv}, left_scale, right_scale}, mlp: {kind: "dense", ff} or null}, ...]

A layer (`parts.DepthMixedBlock`): RMS norm and a short causal convolution in front of each sublayer; a mixer of
two branches side by side (`parts.ParallelMixer`): attention with a distance bias, scores mixed across heads, a
sliding window and a sink (`MixedHeadAttention`), and Griffin's gated linear recurrence (`GatedLinearRecurrence`);
a gated feed-forward with the tanh form of gelu; a per-layer input from the token (`TokenSideInput`); and a learned
mix of all layers' results so far. Embedding: token table plus a learned position table. Tensor names are the
checkpoint's own: `embed`, `pos`, `side.embed`, `l<i>.norm1`, `l<i>.mix.left.q`, ..., `final.norm`, `head`.

Constants the design fixes (not in config.json): the distance slopes 2^(-8 (h + 1) / H), the recurrence's decay
factor 8, gelu's tanh form.
"""
from __future__ import annotations

from dataclasses import dataclass
import json

from ..config.model_config import ConfigError, eos_tuple
from ..config.registry import register_architecture
from ..parts import (CausalConv, DecoderModel, DepthMixedBlock, GatedFeedForward, GatedLinearRecurrence,
                     MixedHeadAttention, OutputHead, ParallelMixer, PositionedEmbedding, RMSNorm, SideTable,
                     TokenSideInput)

SLOPE_BASE = 8.0          # slope_h = 2^(-SLOPE_BASE (h + 1) / H)
RECURRENCE_DECAY = 8.0    # log a = -RECURRENCE_DECAY * r * softplus(lam)


def _need(d, key, where):
    if not isinstance(d, dict) or key not in d:
        raise ConfigError(f"config.json lacks {where}{key!r}")
    return d[key]


def _positive(value, what):
    if isinstance(value, bool) or not isinstance(value, int) or value <= 0:
        raise ConfigError(f"{what} must be a positive integer, found {value!r}")
    return value


@dataclass(frozen=True)
class KanavikConfig:
    architecture: str
    vocab_size: int
    hidden_size: int
    max_position_embeddings: int
    norm_eps: float
    residual_mult: float
    canon_taps: int
    side_dim: int                 # 0: no per-layer token input
    layers: tuple                 # the layer entries of config.json, as immutable JSON text each
    eos_token_ids: tuple = ()

    ARCHITECTURE = "Kanavik"
    MODEL_TYPE = "kanavik"

    @classmethod
    def from_dict(cls, d):
        if d.get("architecture", d.get("model_type")) not in (cls.ARCHITECTURE, cls.MODEL_TYPE):
            raise ConfigError(f"architecture {d.get('architecture')!r} is not {cls.ARCHITECTURE!r}")
        layers = _need(d, "layers", "")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("'layers' must be a non-empty list")
        width = _positive(_need(d, "width", ""), "width")
        for i, layer in enumerate(layers):
            where = f"layers[{i}]."
            if _need(layer, "type", where) != "parallel":
                raise ConfigError(f"layer {i}: mixer type {layer['type']!r} is not built (known: 'parallel')")
            mixer = _need(layer, "mixer", where)
            left, right = _need(mixer, "left", where + "mixer."), _need(mixer, "right", where + "mixer.")
            for key in ("heads", "kv_heads", "dim", "vdim"):
                _positive(_need(left, key, where + "mixer.left."), f"layer {i}: {key}")
            if left["heads"] % left["kv_heads"]:
                raise ConfigError(f"layer {i}: heads must be a multiple of kv_heads")
            if left["heads"] > 32 or max(left["dim"], left["vdim"]) > 256:
                raise ConfigError(f"layer {i}: the attention kernel takes up to 32 heads and head sizes up to 256")
            _need(left, "scale", where + "mixer.left.")
            if left.get("mask") is not None:
                _positive(_need(left["mask"], "size", where + "mixer.left.mask."), f"layer {i}: mask.size")
            for key in ("width", "blocks", "conv"):
                _positive(_need(right, key, where + "mixer.right."), f"layer {i}: {key}")
            if right["width"] % right["blocks"]:
                raise ConfigError(f"layer {i}: the recurrent width must be a multiple of its blocks")
            if right["conv"] > 8:
                raise ConfigError(f"layer {i}: a convolution has at most 8 taps")
            for key in ("left_scale", "right_scale"):
                _need(mixer, key, where + "mixer.")
            mlp = layer.get("mlp")
            if mlp is not None:
                if _need(mlp, "kind", where + "mlp.") != "dense":
                    raise ConfigError(f"layer {i}: feed-forward kind {mlp['kind']!r} is not built (known: 'dense')")
                _positive(_need(mlp, "ff", where + "mlp."), f"layer {i}: ff")
        taps = _positive(_need(_need(d, "canon", ""), "taps", "canon."), "canon.taps")
        if taps > 8:
            raise ConfigError("canon.taps: a convolution has at most 8 taps")
        side = d.get("token_side")
        eps = float(_need(_need(d, "norm", ""), "eps", "norm."))
        if not eps > 0:
            raise ConfigError("norm.eps must be positive")
        return cls(architecture=cls.ARCHITECTURE, vocab_size=_positive(_need(d, "vocab", ""), "vocab"), hidden_size=width,
                   max_position_embeddings=_positive(_need(d, "max_positions", ""), "max_positions"), norm_eps=eps,
                   residual_mult=float(d.get("residual_mult", 1.0)), canon_taps=taps,
                   side_dim=_positive(_need(side, "dim", "token_side."), "token_side.dim") if side else 0,
                   layers=tuple(json.dumps(layer, sort_keys=True) for layer in layers),
                   eos_token_ids=eos_tuple(d.get("eos_token_id")))

    def layer_dicts(self):
        return [json.loads(text) for text in self.layers]

    def to_dict(self):
        d = {"architecture": self.architecture, "vocab": self.vocab_size, "width": self.hidden_size,
             "max_positions": self.max_position_embeddings, "norm": {"eps": self.norm_eps},
             "residual_mult": self.residual_mult, "canon": {"taps": self.canon_taps}, "layers": self.layer_dicts()}
        if self.side_dim:
            d["token_side"] = {"dim": self.side_dim}
        if self.eos_token_ids:
            d["eos_token_id"] = list(self.eos_token_ids)
        return d

    def describe(self):
        return self.to_dict()


def build_kanavik(config: KanavikConfig, packed=True):
    c = config
    C, m, layers = c.hidden_size, c.residual_mult, c.layer_dicts()
    L = len(layers)
    embedding = PositionedEmbedding("embed", c.vocab_size, C, "pos", c.max_position_embeddings, suffix="",
                                    keep=(DepthMixedBlock.HISTORY_TAG, L + 1))
    table = SideTable("side.embed", c.vocab_size, L * c.side_dim) if c.side_dim else None
    blocks = []
    for i, layer in enumerate(layers):
        p = f"l{i}."
        left, right = layer["mixer"]["left"], layer["mixer"]["right"]
        attention = MixedHeadAttention(p + "mix.left.", left["heads"], left["kv_heads"], left["dim"], left["vdim"],
                                       left["scale"], window=(left.get("mask") or {}).get("size"), slope_base=SLOPE_BASE)
        recurrence = GatedLinearRecurrence(p + "mix.right.", right["width"], right["blocks"], right["conv"],
                                           decay=RECURRENCE_DECAY)
        mixer = ParallelMixer(C, [attention, recurrence], [layer["mixer"]["left_scale"], layer["mixer"]["right_scale"]],
                              out_scale=m)
        mixer_in = CausalConv(p + "canon1", C, c.canon_taps, "canon1", identity=1.0,
                              norm=RMSNorm(p + "norm1", C, c.norm_eps, suffix=""))
        ffn = ffn_in = None
        if layer.get("mlp"):
            ffn = GatedFeedForward([p + "mlp.gate", p + "mlp.up", p + "mlp.down"], C, layer["mlp"]["ff"], out_scale=m,
                                   suffix="")
            ffn_in = CausalConv(p + "canon2", C, c.canon_taps, "canon2", identity=1.0,
                                norm=RMSNorm(p + "norm2", C, c.norm_eps, suffix=""))
        side = TokenSideInput(p + "side.", table, i, C, c.side_dim, c.norm_eps, owns_table=i == 0) if table else None
        unused = () if ffn is not None else (p + "norm2", p + "canon2")
        blocks.append(DepthMixedBlock(i, L, C, mixer_in, mixer, ffn_in, ffn, side, side_mult=m, mix_name=p + "dwa",
                                      unused_names=unused))
    final_norm = RMSNorm("final.norm", C, c.norm_eps, suffix="")
    head = OutputHead("head", c.vocab_size, C, suffix="")
    return DecoderModel(c, embedding, blocks, final_norm, head)


register_architecture(KanavikConfig.ARCHITECTURE, KanavikConfig.MODEL_TYPE, KanavikConfig, build_kanavik, replace=True)

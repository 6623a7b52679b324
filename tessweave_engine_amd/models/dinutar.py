"""The Dinutar decoder: its typed configuration and its model assembled from parts.

config.json gives every size and every constant that differs between models of the design:

    architecture "Dinutar", vocab, width, norm.eps, postln_alpha,
    embedding: {scale, bigram: {buckets, mul_prev, mul_cur}},
    layers: [{type: "latent_attention", mixer: {heads, dim, rot_dim, vdim, kv_rank, scale, rot: {base, dims[, scaling:
              {factor, original, fast, slow}]}[, kv_from: j]}, mlp: {kind: "dense", ff} or null},
             {type: "retention", mixer: {heads, dim, vdim, decay: [..], rot: {...}}, mlp: ...}, ...]

Embedding (`parts.HashedPairEmbedding`): the token's row times a scale plus a row of a second table chosen by a hash
of (previous token, token), then an RMS norm. A layer (`parts.PostNormBlock`) norms AFTER each sum,
x <- norm(alpha x + ls * sublayer(x)), with a learned scale per channel on the sublayer's result. Mixers: attention
over a cached latent with a rotated key part shared by all heads (`parts.LatentAttention`; a layer with `kv_from`
reads the cache slot of an earlier layer instead of writing one), or retention (`parts.Retention`). Feed-forward:
down(relu(up(h))^2) (`parts.ReluSquaredFeedForward`) or none. Output: RMS norm, then the embedding table itself as
the head. Tensor names are the checkpoint's own: `embed`, `bigram`, `embed.norm`, `l<i>.norm1`, `l<i>.mix.q`, ...,
`l<i>.ls1`, `final.norm`.

Constants the design fixes (not in config.json): retention's keys are multiplied by dim^-1/2; the stretched rotary
encoding's cos and sin grow by 0.1 ln(factor) + 1 (`parts.RotaryEmbedding(stretch=)`); the feed-forward's activation.
"""
from __future__ import annotations

from dataclasses import dataclass
import json

from ..config.model_config import ConfigError, eos_tuple
from ..config.registry import register_architecture
from ..parts import (DecoderModel, HashedPairEmbedding, LatentAttention, LayerRun, NoPositionEncoding, OutputHead,
                     PostNormBlock, ReluSquaredFeedForward, Retention, RMSNorm, RotaryEmbedding)

MIXERS = ("latent_attention", "retention")
NO_POSITION_LIMIT = 1 << 30      # the design has no learned positions: nothing bounds a request's length but the cache


def _need(d, key, where):
    if not isinstance(d, dict) or key not in d:
        raise ConfigError(f"config.json lacks {where}{key!r}")
    return d[key]


def _positive(value, what):
    if isinstance(value, bool) or not isinstance(value, int) or value <= 0:
        raise ConfigError(f"{what} must be a positive integer, found {value!r}")
    return value


def _check_rot(rot, limit, where):
    dims = _positive(_need(rot, "dims", where), where + "dims")
    if dims % 2 or dims > limit:
        raise ConfigError(f"{where}dims must be even and at most {limit}")
    if not float(_need(rot, "base", where)) > 1:
        raise ConfigError(f"{where}base must be greater than 1")
    scaling = rot.get("scaling")
    if scaling is not None:
        for key in ("factor", "original", "fast", "slow"):
            if not float(_need(scaling, key, where + "scaling.")) > 0:
                raise ConfigError(f"{where}scaling.{key} must be positive")


@dataclass(frozen=True)
class DinutarConfig:
    architecture: str
    vocab_size: int
    hidden_size: int
    norm_eps: float
    postln_alpha: float
    embedding_scale: float
    pair_buckets: int
    pair_mul_prev: int
    pair_mul_cur: int
    layers: tuple                 # the layer entries of config.json, as immutable JSON text each
    max_position_embeddings: int = NO_POSITION_LIMIT
    eos_token_ids: tuple = ()

    ARCHITECTURE = "Dinutar"
    MODEL_TYPE = "dinutar"

    @classmethod
    def from_dict(cls, d):
        if d.get("architecture", d.get("model_type")) not in (cls.ARCHITECTURE, cls.MODEL_TYPE):
            raise ConfigError(f"architecture {d.get('architecture')!r} is not {cls.ARCHITECTURE!r}")
        layers = _need(d, "layers", "")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("'layers' must be a non-empty list")
        for i, layer in enumerate(layers):
            where = f"layers[{i}]."
            kind = _need(layer, "type", where)
            if kind not in MIXERS:
                raise ConfigError(f"layer {i}: mixer type {kind!r} is not built (known: {', '.join(MIXERS)})")
            m = _need(layer, "mixer", where)
            for key in ("heads", "dim", "vdim"):
                _positive(_need(m, key, where + "mixer."), f"layer {i}: {key}")
            if kind == "latent_attention":
                for key in ("rot_dim", "kv_rank"):
                    _positive(_need(m, key, where + "mixer."), f"layer {i}: {key}")
                _need(m, "scale", where + "mixer.")
                _check_rot(_need(m, "rot", where + "mixer."), m["rot_dim"], where + "mixer.rot.")
                if max(m["dim"] + m["rot_dim"], m["vdim"]) > 256:
                    raise ConfigError(f"layer {i}: the attention kernels take dim + rot_dim and vdim up to 256")
                source = m.get("kv_from")
                if source is not None:
                    if isinstance(source, bool) or not isinstance(source, int) or not 0 <= source < i:
                        raise ConfigError(f"layer {i}: kv_from must name an earlier layer")
                    other = layers[source]
                    om = other.get("mixer", {})
                    if other.get("type") != "latent_attention" or om.get("kv_from") is not None:
                        raise ConfigError(f"layer {i}: kv_from must name a latent attention layer with a latent of its own")
                    if (om.get("kv_rank"), om.get("rot_dim"), om.get("rot")) != (m["kv_rank"], m["rot_dim"], m["rot"]):
                        raise ConfigError(f"layer {i}: kv_rank, rot_dim and rot must equal those of layer {source}")
            else:
                if m["dim"] > 256:
                    raise ConfigError(f"layer {i}: the retention kernels take key sizes up to 256")
                decay = _need(m, "decay", where + "mixer.")
                if not isinstance(decay, list) or len(decay) != m["heads"] or not all(0 < float(v) <= 1 for v in decay):
                    raise ConfigError(f"layer {i}: decay must list one factor in (0, 1] per head")
                if m.get("rot") is not None:
                    _check_rot(m["rot"], m["dim"], where + "mixer.rot.")
            mlp = layer.get("mlp")
            if mlp is not None:
                if _need(mlp, "kind", where + "mlp.") != "dense":
                    raise ConfigError(f"layer {i}: feed-forward kind {mlp['kind']!r} is not built (known: 'dense')")
                _positive(_need(mlp, "ff", where + "mlp."), f"layer {i}: ff")
        eps = float(_need(_need(d, "norm", ""), "eps", "norm."))
        if not eps > 0:
            raise ConfigError("norm.eps must be positive")
        emb = _need(d, "embedding", "")
        pair = _need(emb, "bigram", "embedding.")
        for key in ("mul_prev", "mul_cur"):
            v = _need(pair, key, "embedding.bigram.")
            if isinstance(v, bool) or not isinstance(v, int) or v < 0:
                raise ConfigError(f"embedding.bigram.{key} must be an integer that is not negative")
        return cls(architecture=cls.ARCHITECTURE, vocab_size=_positive(_need(d, "vocab", ""), "vocab"),
                   hidden_size=_positive(_need(d, "width", ""), "width"), norm_eps=eps,
                   postln_alpha=float(_need(d, "postln_alpha", "")), embedding_scale=float(_need(emb, "scale", "embedding.")),
                   pair_buckets=_positive(_need(pair, "buckets", "embedding.bigram."), "embedding.bigram.buckets"),
                   pair_mul_prev=pair["mul_prev"], pair_mul_cur=pair["mul_cur"],
                   layers=tuple(json.dumps(layer, sort_keys=True) for layer in layers),
                   eos_token_ids=eos_tuple(d.get("eos_token_id")))

    def layer_dicts(self):
        return [json.loads(text) for text in self.layers]

    def to_dict(self):
        d = {"architecture": self.architecture, "vocab": self.vocab_size, "width": self.hidden_size,
             "norm": {"eps": self.norm_eps}, "postln_alpha": self.postln_alpha,
             "embedding": {"scale": self.embedding_scale, "bigram": {"buckets": self.pair_buckets,
                                                                     "mul_prev": self.pair_mul_prev,
                                                                     "mul_cur": self.pair_mul_cur}},
             "layers": self.layer_dicts()}
        if self.eos_token_ids:
            d["eos_token_id"] = list(self.eos_token_ids)
        return d

    def describe(self):
        return self.to_dict()


def build_dinutar(config: DinutarConfig, packed=True):
    c = config
    C, layers = c.hidden_size, c.layer_dicts()
    encodings = {}

    def rotary(rot, size):
        """One part per distinct encoding: its tables are formed once a step for all layers that share it."""
        if rot is None:
            return NoPositionEncoding()
        scaling = rot.get("scaling")
        stretch = (scaling["factor"], scaling["original"], scaling["fast"], scaling["slow"]) if scaling else None
        key = (size, float(rot["base"]), int(rot["dims"]), stretch)
        if key not in encodings:
            encodings[key] = RotaryEmbedding(size, rot["base"], rot["dims"], stretch=stretch)
        return encodings[key]

    embedding = HashedPairEmbedding("embed", c.vocab_size, C, "bigram", c.pair_buckets, c.pair_mul_prev, c.pair_mul_cur,
                                    RMSNorm("embed.norm", C, c.norm_eps, suffix=""), scale=c.embedding_scale, suffix="")
    blocks, schedule, slot_of = [], [], {}
    for i, layer in enumerate(layers):
        p, m = f"l{i}.", layer["mixer"]
        if layer["type"] == "latent_attention":
            source = m.get("kv_from")
            mixer = LatentAttention(p + "mix.", C, m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["scale"],
                                    rotary(m["rot"], m["rot_dim"]), c.norm_eps, own_latent=source is None)
        else:
            source = None
            mixer = Retention(p + "mix.", C, m["heads"], m["dim"], m["vdim"], m["decay"], rotary(m.get("rot"), m["dim"]),
                              c.norm_eps)
        ffn = ffn_norm = None
        if layer.get("mlp"):
            ffn = ReluSquaredFeedForward([p + "mlp.up", p + "mlp.down"], C, layer["mlp"]["ff"], suffix="")
            ffn_norm = RMSNorm(p + "norm2", C, c.norm_eps, suffix="")
        blocks.append(PostNormBlock(C, mixer, RMSNorm(p + "norm1", C, c.norm_eps, suffix=""), ffn, ffn_norm,
                                    alpha=c.postln_alpha, mixer_scale_name=p + "ls1", ffn_scale_name=p + "ls2"))
        if source is None:
            slot_of[i] = len(slot_of)
            schedule.append(LayerRun(i, slot_of[i]))
        else:
            schedule.append(LayerRun(i, slot_of[source], writes_cache=False))
    final_norm = RMSNorm("final.norm", C, c.norm_eps, suffix="")
    head = OutputHead("head", c.vocab_size, C, tied_to=embedding, suffix="")
    return DecoderModel(c, embedding, blocks, final_norm, head, schedule=schedule)


register_architecture(DinutarConfig.ARCHITECTURE, DinutarConfig.MODEL_TYPE, DinutarConfig, build_dinutar, replace=True)

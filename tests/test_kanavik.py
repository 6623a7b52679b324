"""The Kanavik design without a GPU: configuration, registry, tensor names, cache needs, and the plain
implementation's mechanisms against closed forms (so that the oracle the GPU tests use is itself pinned)."""
import json
import math

import pytest
import torch

import plain_kanavik as plain
from kanavik_util import CONFIGS, make_weights, tensor_shapes, write_folder


@pytest.mark.parametrize("name", list(CONFIGS))
def test_config_registry_and_tensor_names(name, tmp_path):
    from tessweave_engine_amd.config import build_model, config_from_dict, read_model_config
    c = CONFIGS[name]
    config = config_from_dict(c)
    assert config.architecture == "Kanavik" and config.vocab_size == c["vocab"]
    assert config_from_dict(config.to_dict()) == config
    model = build_model(config)
    specs = {s.name: s.shape for s in model.tensor_specs() if s.optional_alias_of is None}
    assert specs == tensor_shapes(c)
    # a layer without a feed-forward may still bring its second norm and convolution: accepted, never required
    spare = sorted(s.name for s in model.tensor_specs() if s.optional_alias_of is not None)
    assert spare == sorted(f"l{i}.{t}" for i, lay in enumerate(c["layers"]) if not lay["mlp"] for t in ("norm2", "canon2"))
    folder = write_folder(tmp_path, c, make_weights(c, 0))
    assert read_model_config(folder) == config


def test_config_rejections():
    from tessweave_engine_amd.config import ConfigError, config_from_dict
    base = json.loads(json.dumps(CONFIGS["odd"]))
    for change in (lambda c: c["layers"][0].__setitem__("type", "other"),
                   lambda c: c["layers"][1]["mixer"]["left"].__setitem__("kv_heads", 4),
                   lambda c: c["layers"][0]["mixer"]["right"].__setitem__("blocks", 5),
                   lambda c: c["layers"][0]["mlp"].__setitem__("kind", "experts"),
                   lambda c: c.pop("canon"),
                   lambda c: c["norm"].__setitem__("eps", 0)):
        c = json.loads(json.dumps(base))
        change(c)
        with pytest.raises(ConfigError):
            config_from_dict(c)


def test_cache_needs_and_state_slots():
    """Each layer's cache slot: pages for the window's keys and values (sizes rounded up to 16 on the device), the
    recurrence's state, and the last inputs of its convolutions twice over."""
    from tessweave_engine_amd.cache import CacheManager
    from tessweave_engine_amd.config import build_model, config_from_dict
    c = CONFIGS["odd"]
    layout = build_model(config_from_dict(c)).cache_layout()
    assert [(g.spec.kv_heads, g.spec.head_dim, g.spec.value_dim, g.spec.window) for g in layout.groups] == \
        [(4, 32, 48, 7), (2, 32, 16, 33), (1, 80, 96, 1000)]
    states = dict(layout.needs[0].states)
    assert states["recurrent.s"].shape == (36,) and states["recurrent.conv"].shape == (2, 3, 36)
    assert states["canon1"].shape == (2, 3, 96) and states["canon2"].shape == (2, 3, 96)
    assert "canon2" not in dict(layout.needs[1].states)            # the layer without a feed-forward
    assert dict(layout.needs[2].states)["recurrent.conv"].shape == (2, 1, 24)     # one tap: nothing to keep, one row held
    assert not layout.shares_prefixes
    m = CacheManager(layout, 8, 16, 2)
    a, b = m.open("a"), m.open("b")
    assert {a.state_slot, b.state_slot} == {0, 1} and a.steps == 0
    m.ensure(a, 40)
    m.advance(a, 40)
    assert a.held(0) == 1 and a.held(1) == 4 and a.held(2) == 5    # what queries from position 40 on can still see
    m.close(a)
    assert m.open("c").state_slot == a.state_slot
    m.check()


def test_plain_mechanisms_against_closed_forms():
    g = torch.Generator().manual_seed(0)
    # convolution: the last column meets the current token; nothing from the future
    h = torch.randn(6, 3, generator=g, dtype=torch.float64)
    w = torch.tensor([[0.0, 0.0, 1.0]] * 3, dtype=torch.float64)
    assert torch.equal(plain.causal_conv(h, w), h)
    w = torch.tensor([[1.0, 0.0, 0.0]] * 3, dtype=torch.float64)
    assert torch.equal(plain.causal_conv(h, w)[2:], h[:-2]) and plain.causal_conv(h, w)[:2].abs().sum() == 0
    # recurrence: constant gates give a geometric series; a and sqrt(1 - a^2) from log a = -8 r softplus(lam)
    lam = torch.tensor([0.3], dtype=torch.float64)
    r = torch.full((5, 1), 0.25, dtype=torch.float64)
    a = math.exp(-8 * 0.25 * math.log1p(math.exp(0.3)))
    S = plain.gated_recurrence(torch.ones(5, 1, dtype=torch.float64), r, torch.full((5, 1), 0.5, dtype=torch.float64), lam)
    want = [math.sqrt(1 - a * a) * 0.5 * sum(a ** k for k in range(t + 1)) for t in range(5)]
    assert torch.allclose(S[:, 0], torch.tensor(want, dtype=torch.float64))
    # attention: zero queries, identity mixing, no sink mass: the mean of the window's values weighted by the slopes
    T, H = 9, 2
    v = torch.randn(T, 1, 4, generator=g, dtype=torch.float64)
    out = plain.mixed_head_attention(torch.zeros(T, H, 4, dtype=torch.float64), torch.zeros(T, 1, 4, dtype=torch.float64), v, 1.0, 3,
                                     torch.eye(H, dtype=torch.float64), torch.full((H,), -1e9, dtype=torch.float64))
    slopes = [2.0 ** (-8 * (h + 1) / H) for h in range(H)]
    for hd in range(H):
        wts = torch.tensor([math.exp(-slopes[hd] * d) for d in (2, 1, 0)], dtype=torch.float64)
        assert torch.allclose(out[8, hd], (wts[:, None] * v[6:9, 0]).sum(0) / wts.sum())
    # the sink counts once, with no value: a sink equal to the only score halves the output
    one = plain.mixed_head_attention(torch.zeros(1, 1, 4, dtype=torch.float64), torch.zeros(1, 1, 4, dtype=torch.float64), v[:1], 1.0, 3,
                                     torch.eye(1, dtype=torch.float64), torch.zeros(1, dtype=torch.float64))
    assert torch.allclose(one[0, 0], v[0, 0] / 2)
    # mixing happens before the softmax: swapping the heads' rows of the matrix swaps the heads' outputs
    q = torch.randn(T, H, 4, generator=g, dtype=torch.float64)
    k = torch.randn(T, 1, 4, generator=g, dtype=torch.float64)
    sink = torch.zeros(H, dtype=torch.float64)
    talk = torch.randn(H, H, generator=g, dtype=torch.float64)
    a1 = plain.mixed_head_attention(q, k, v, 0.5, 4, talk, sink)
    a2 = plain.mixed_head_attention(q, k, v, 0.5, 4, talk.flip(0), sink)
    assert torch.allclose(a1, a2.flip(1))


def test_plain_model_is_causal_and_uses_every_part():
    c = CONFIGS["one"]
    w = make_weights(c, 3)
    toks = torch.randint(0, c["vocab"], (12,), generator=torch.Generator().manual_seed(1)).tolist()
    full = plain.forward(c, w, toks)
    assert torch.allclose(plain.forward(c, w, toks[:7]), full[:7], atol=1e-9)
    for name in ("pos", "side.embed", "l0.dwa", "l0.mix.left.talk", "l0.mix.left.sink", "l0.mix.right.lam", "l0.mix.right.conv",
                 "l0.side.norm", "l0.mix.right.ri"):
        changed = dict(w)
        changed[name] = (w[name].float() * 1.5 + 0.25).to(torch.bfloat16)
        assert (plain.forward(c, changed, toks) - full).abs().max() > 1e-4, name

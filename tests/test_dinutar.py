"""The Dinutar design without a GPU: configuration, registry, tensor names, cache needs and schedule, and the plain
implementation's mechanisms against closed forms (so that the oracle the GPU tests use is itself pinned)."""
import json
import math

import pytest
import torch

import plain_dinutar as plain
from dinutar_util import CONFIGS, make_weights, tensor_shapes, write_folder


@pytest.mark.parametrize("name", list(CONFIGS))
def test_config_registry_and_tensor_names(name, tmp_path):
    from tessweave_engine_amd.config import build_model, config_from_dict, read_model_config
    c = CONFIGS[name]
    config = config_from_dict(c)
    assert config.architecture == "Dinutar" and config.vocab_size == c["vocab"]
    assert config_from_dict(config.to_dict()) == config
    model = build_model(config)
    specs = {s.name: s.shape for s in model.tensor_specs() if s.optional_alias_of is None}
    assert specs == tensor_shapes(c)
    folder = write_folder(tmp_path, c, make_weights(c, 0))
    assert read_model_config(folder) == config


def test_config_rejections():
    from tessweave_engine_amd.config import ConfigError, config_from_dict
    base = json.loads(json.dumps(CONFIGS["odd"]))
    for change in (lambda c: c["layers"][0].__setitem__("type", "other"),
                   lambda c: c["layers"][1]["mixer"].__setitem__("decay", [0.5]),
                   lambda c: c["layers"][2]["mixer"].__setitem__("kv_from", 2),
                   lambda c: c["layers"][2]["mixer"].__setitem__("kv_from", 1),
                   lambda c: c["layers"][2]["mixer"].__setitem__("kv_rank", 32),
                   lambda c: c["layers"][0]["mixer"]["rot"].__setitem__("dims", 7),
                   lambda c: c["layers"][0]["mlp"].__setitem__("kind", "experts"),
                   lambda c: c.pop("embedding"),
                   lambda c: c.pop("postln_alpha"),
                   lambda c: c["norm"].__setitem__("eps", 0)):
        c = json.loads(json.dumps(base))
        change(c)
        with pytest.raises(ConfigError):
            config_from_dict(c)


def test_cache_layout_and_schedule():
    """Layers with a latent of their own page it (one key/value head: latent and rotated part, each rounded up to 16;
    values the latent's size), readers run on the writer's slot, retention layers hold a float32 state, and the
    embedding's last token has a slot of its own behind the layers'."""
    from tessweave_engine_amd.config import build_model, config_from_dict
    model = build_model(config_from_dict(CONFIGS["wide"]))
    layout = model.cache_layout()
    runs = [(r.block, r.cache_slot, r.writes_cache) for r in model.schedule]
    assert runs == [(0, 0, True), (1, 1, True), (2, 2, True), (3, 1, False), (4, 3, True), (5, 2, False)]
    assert layout.needs[1].paged.kv_heads == 1 and layout.needs[1].paged.head_dim == 96 + 32 and layout.needs[1].paged.value_dim == 96
    assert layout.needs[2].paged.head_dim == 32 + 16 and len(layout.groups) == 2
    assert dict(layout.needs[0].states)["retention.s"].shape == (1, 64, 128)
    assert dict(layout.needs[4].states)["last_token"].dtype == "int32" and model.embedding.cache_slot == 4
    assert not layout.shares_prefixes


def test_pair_rows_and_first_token():
    rows = plain.bigram_rows([5, 9, 9, 2], 7, 3, 4)
    assert rows == [7, (5 * 3 + 9 * 4) % 7, (9 * 3 + 9 * 4) % 7, (9 * 3 + 2 * 4) % 7]
    assert plain.bigram_rows([0], 11, 1, 1) == [11]


def test_stretched_frequencies():
    """Pairs that turn often inside the original context keep their frequency, slow ones are divided by the factor,
    and without stretching the frequencies are base^(-2i/dims) with a magnitude of one."""
    f, mag = plain.rotary_frequencies(8, 100.0)
    assert mag == 1.0 and torch.allclose(f, torch.tensor([1.0, 100 ** -0.25, 0.1, 100 ** -0.75], dtype=torch.float64))
    scaling = {"factor": 4.0, "original": 64, "fast": 16.0, "slow": 1.0}
    g, mag = plain.rotary_frequencies(16, 10000.0, scaling)
    f, _ = plain.rotary_frequencies(16, 10000.0)
    assert mag == pytest.approx(0.1 * math.log(4.0) + 1.0)
    lo = max(math.floor(16 * math.log(64 / (2 * math.pi * 16)) / (2 * math.log(1e4))), 0)
    hi = min(math.ceil(16 * math.log(64 / (2 * math.pi * 1)) / (2 * math.log(1e4))), 15)
    assert torch.allclose(g[:lo + 1], f[:lo + 1]) and torch.allclose(g[hi:], f[hi:] / 4.0)
    assert all(f[i] / 4.0 < g[i] < f[i] for i in range(lo + 1, hi))


def test_rotation_is_a_turn_of_pairs():
    x = torch.randn(5, 2, 12, dtype=torch.float64)
    y = plain.rotate(x, torch.arange(5), 8, 50.0)
    assert torch.equal(y[..., 8:], x[..., 8:]) and torch.equal(y[0], x[0])
    assert torch.allclose((y[..., :4] ** 2 + y[..., 4:8] ** 2), (x[..., :4] ** 2 + x[..., 4:8] ** 2))
    # scores depend on the distance alone
    q, k = torch.randn(1, 1, 8, dtype=torch.float64), torch.randn(1, 1, 8, dtype=torch.float64)
    a = (plain.rotate(q, torch.tensor([7]), 8, 50.0) * plain.rotate(k, torch.tensor([3]), 8, 50.0)).sum()
    b = (plain.rotate(q, torch.tensor([14]), 8, 50.0) * plain.rotate(k, torch.tensor([10]), 8, 50.0)).sum()
    assert a.item() == pytest.approx(b.item())


def test_retention_is_a_decayed_sum():
    """With no rotation the state's closed form is o_t = sum_j decay^(t - j) (q_t . k_j) v_j / sqrt(D)."""
    T, C, H, D, E = 9, 6, 2, 4, 3
    g = torch.Generator().manual_seed(1)
    h = torch.randn(T, C, generator=g, dtype=torch.float64)
    wq, wk = torch.randn(H * D, C, generator=g, dtype=torch.float64), torch.randn(H * D, C, generator=g, dtype=torch.float64)
    wv, wg = torch.randn(H * E, C, generator=g, dtype=torch.float64), torch.randn(H * E, C, generator=g, dtype=torch.float64)
    wo = torch.eye(H * E, dtype=torch.float64)
    decay = [0.5, 1.0]
    got = plain.retention(h, wq, wk, wv, wg, wo, H, D, E, decay, 1e-6, torch.arange(T), None)
    q, k, v = (h @ wq.T).view(T, H, D), (h @ wk.T).view(T, H, D) / 2.0, (h @ wv.T).view(T, H, E)
    o = torch.zeros(T, H, E, dtype=torch.float64)
    for t in range(T):
        for j in range(t + 1):
            for a in range(H):
                o[t, a] += decay[a] ** (t - j) * (q[t, a] @ k[j, a]) * v[j, a]
    want = plain.rms_unit(o, 1e-6).reshape(T, H * E) * torch.nn.functional.silu(h @ wg.T)
    assert torch.allclose(got, want, atol=1e-6)


def test_latent_attention_reads_another_layers_latent():
    """A reader with the writer's own matrices gives the writer's result; the first token attends to itself alone."""
    c = CONFIGS["one"]
    w = {k: v.double() for k, v in make_weights(c, 3).items()}
    m = c["layers"][0]["mixer"]
    T = 6
    h = torch.randn(T, c["width"], dtype=torch.float64)
    pos = torch.arange(T)
    lat, shared = plain.latent_from(h, w["l0.mix.dkv"], w["l0.mix.dkv.norm"], m["kv_rank"], 1e-5, pos, m["rot"])
    out = plain.latent_attention(h, lat, shared, w["l0.mix.q"], w["l0.mix.uk"], w["l0.mix.uv"], w["l0.mix.o"], m["heads"],
                                 m["dim"], m["rot_dim"], m["vdim"], m["scale"], pos, m["rot"])
    first = (lat[:1] @ w["l0.mix.uv"].T) @ w["l0.mix.o"].T
    assert torch.allclose(out[:1], first, atol=1e-9)
    assert torch.allclose((lat ** 2).mean(-1) / (w["l0.mix.dkv.norm"] ** 2).mean(), torch.ones(T, dtype=torch.float64), rtol=0.8)


def test_relu_squared():
    h = torch.tensor([[1.0, -2.0]], dtype=torch.float64)
    up = torch.tensor([[1.0, 0.0], [0.0, 1.0], [2.0, 0.0]], dtype=torch.float64)
    down = torch.tensor([[1.0, 1.0, 1.0]], dtype=torch.float64)
    assert plain.relu_squared_ff(h, up, down).item() == 1.0 + 0.0 + 4.0


def test_command_line_inspect_and_random_weights(tmp_path, capsys):
    """`random-weights` writes a folder for the design from its config.json alone; `inspect` reports the cache groups
    (one key/value head of latent + rotated part, values of the latent's size) and what a request holds besides pages."""
    from safetensors import safe_open
    from tessweave_engine_amd.cli import main
    c = CONFIGS["wide"]
    (tmp_path / "config.json").write_text(json.dumps(c))
    out = tmp_path / "model"
    assert main(["random-weights", str(tmp_path / "config.json"), str(out), "--seed", "3"]) == 0
    with safe_open(str(out / "model.safetensors"), framework="pt") as f:
        assert {k: tuple(f.get_slice(k).get_shape()) for k in f.keys()} == tensor_shapes(c)
    capsys.readouterr()
    assert main(["inspect", str(out), "--kv-blocks", "10", "--block-size", "16"]) == 0
    report = json.loads(capsys.readouterr().out)
    groups = sorted((g["layers"], g["kv_heads"], g["head_dim"], g.get("value_dim")) for g in report["cache_groups"])
    assert groups == [(1, 1, 48, 32), (1, 1, 128, 96)]
    states = 4 * (1 * 64 * 128 + 4 * 16 * 16) + 4 * 2
    assert report["state_bytes_per_request"] == states

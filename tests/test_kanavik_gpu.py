"""The Kanavik design on the GPU against the plain implementation (`plain_kanavik.py`).

Mechanisms alone (each kernel against the plain function of the same name, with inputs made so that a
fault shows: one key far away that carries all the weight, keys just inside and just outside a window,
at page borders, a sink that takes most of the mass, state that is carried over portions and reused
slots), then whole models through the package's loader, cache manager and step function: prefill
against token-by-token decoding, portions down to two tokens, unequal batches against each request
alone, few pages and slots that are freed and used again, long decoding from HIP graphs, and greedy
generation through the scheduler.

Bars: float32 rows must agree with the float64 plain implementation to 2e-5 of the logits' spread (the
kernels sum in other orders); bfloat16 to 3 % of it (bfloat16 rounds to 0.4 %, a few dozen roundings
deep).
"""
import math

import numpy as np
import pytest
import torch

import plain_kanavik as plain
from kanavik_util import CONFIGS, Driver, make_weights, row_error, write_folder

pytestmark = pytest.mark.gpu

BAR = {"float32": 2e-5, "bfloat16": 3e-2}


def tdtype(name):
    return getattr(torch, name)


# ---------------------------------------------------------------------------------------------------------
# mechanisms alone
# ---------------------------------------------------------------------------------------------------------

def paged(keys, values, page, order):
    """keys [T, G, D], values [T, G, E] laid into pages in the given physical order; returns the kernel's
    tensors and the block table row."""
    T, G, D = keys.shape
    E = values.shape[2]
    blocks = (T + page - 1) // page
    n_pages = max(order[:blocks]) + 1
    kp = torch.full((n_pages + 1, G, page, D), float("nan"), dtype=keys.dtype, device=keys.device)
    vp = torch.full((n_pages + 1, G, E, page), float("nan"), dtype=keys.dtype, device=keys.device)
    for b in range(blocks):
        lo, hi = b * page, min(T, (b + 1) * page)
        kp[order[b], :, :hi - lo] = keys[lo:hi].transpose(0, 1)
        vp[order[b], :, :, :hi - lo] = values[lo:hi].permute(1, 2, 0)
    return kp, vp, torch.tensor([order[:blocks]], dtype=torch.int32, device=keys.device)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H,G,D,E,window,T,q_len,page", [
    (4, 2, 32, 16, 9, 70, 70, 8),          # whole prompt, window crosses pages
    (3, 3, 16, 48, 0, 45, 13, 4),          # no window, a portion behind cached keys
    (20, 4, 16, 32, 33, 50, 50, 16),       # two heads a wave
    (32, 8, 128, 64, 40, 90, 90, 16),      # so many long heads that a tile's queries stay in memory
    (2, 1, 80, 128, 17, 300, 1, 16),       # decode
    (6, 2, 64, 96, 0, 700, 1, 32),         # decode over many keys: several key ranges
    (5, 1, 32, 48, 200, 400, 150, 16),     # a portion whose tiles' keys are cut into ranges
])
def test_mixed_head_attention(device, dtype, H, G, D, E, window, T, q_len, page):
    from tessweave_engine_amd.kernels import ops
    g = torch.Generator().manual_seed(H * 1000 + T)
    dt = tdtype(dtype)
    q = torch.randn(T, H, D, generator=g)
    k = torch.randn(T, G, D, generator=g)
    v = torch.randn(T, G, E, generator=g)
    # one far key (position 3) answers the last query loudly in the last head (whose distance slope is the
    # smallest), as far as the window lets it
    unit = q[T - 1, H - 1] / q[T - 1, H - 1].norm()
    k[3, G - 1] = 12.0 * unit
    q[T - 1, H - 1] *= 3.0
    # the keys just inside and just outside the last query's window are loud too
    if window and T > window:
        for j in (T - window, T - window - 1):
            k[j, G - 1] = 9.0 * unit
    q, k, v = (t.to(dt).float() for t in (q, k, v))
    talk = (torch.eye(H) + 0.5 * torch.randn(H, H, generator=g))
    sink = torch.randn(H, generator=g)
    sink[0] = 6.0                                          # one head whose sink takes most of the mass
    scale = 0.3 / math.sqrt(D)
    want = plain.mixed_head_attention(q.double(), k.double(), v.double(), scale, window or 10 ** 9, talk.double(),
                                      sink.double())[T - q_len:].reshape(q_len, H * E)
    order = list(reversed(range((T + page - 1) // page)))  # pages in reverse physical order
    kp, vp, table = paged(k.to(dt).to(device), v.to(dt).to(device), page, order)
    qd = q[T - q_len:].reshape(q_len, H * D).to(dt).to(device)
    out = torch.empty(q_len, H * E, dtype=dt, device=device)
    q_start = torch.tensor([0, q_len], dtype=torch.int32, device=device)
    kv_len = torch.tensor([T], dtype=torch.int32, device=device)
    slopes = torch.tensor(plain.distance_slopes(H).tolist(), dtype=torch.float32, device=device)
    splits, ws = 1, None
    if q_len == 1:
        splits = ops.attn_mixed_splits(1, T)
        assert (splits > 1) == (T >= 128)
        ws = torch.empty(ops.attn_mixed_workspace_floats(1, 1, H, E, splits), dtype=torch.float32, device=device)
    elif T >= 256:
        splits = 3                                         # a prompt portion whose tiles' keys are cut into ranges
        ws = torch.full((ops.attn_mixed_workspace_floats(1, q_len, H, E, splits),), float("nan"), device=device)
    ops.attn_mixed(qd, kp, vp, table, q_start, kv_len, 0, 1, q_len, out, H, G, scale, window=window,
                   talk=talk.to(device), sink=sink.to(device), slopes=slopes, out_scale=0.5, splits=splits, workspace=ws)
    got = out.float().cpu().numpy() / 0.5
    assert np.isfinite(got).all()
    err = row_error(got, want.numpy()).max()
    assert err < (1e-5 if dtype == "float32" else 2e-2), err
    # without the far key's weight the last row would differ: the test can see it
    if not window or T <= window:
        blind = plain.mixed_head_attention(q.double()[4:], k.double()[4:], v.double()[4:], scale, 10 ** 9, talk.double(),
                                           sink.double())[-1].reshape(H * E)
        assert row_error(blind.numpy()[None], want.numpy()[-1:]).max() > 0.05


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("taps,norm,C", [(3, True, 40), (4, False, 40), (1, True, 38), (2, False, 38), (8, True, 38)])
def test_causal_conv_over_portions_and_reused_slots(device, dtype, taps, norm, C):
    """Sequences in portions of 1 to 9 tokens, two at a time, in state slots that were used before."""
    from tessweave_engine_amd.kernels import ops
    g = torch.Generator().manual_seed(taps * 7 + norm)
    dt = tdtype(dtype)
    w = torch.randn(C, taps, generator=g)
    bias = None if norm else torch.randn(C, generator=g)
    nw = 1 + 0.3 * torch.randn(C, generator=g)
    state = torch.full((3, 2, max(taps - 1, 1), C), float("nan"), device=device)    # stale contents must not matter ...
    for round_ in range(2):
        seqs = [torch.randn(n, C, generator=g) for n in (23, 17)]
        if not norm:
            seqs = [s.to(dt).float() for s in seqs]
        slots = [2, 0] if round_ == 0 else [0, 2]
        state[slots] = 0                                                           # ... once a slot is zeroed at opening
        want = []
        for s in seqs:
            v = plain.rms_norm(s.double(), nw.double(), 1e-5) if norm else s.double()
            want.append((v if norm else 0) + plain.causal_conv(v, w.double()) + (0 if norm else bias.double()))
        at, steps, got = [0, 0], [0, 0], [[], []]
        sizes = [1, 2, 9, 3, 1, 1, 5, 2, 4, 6]
        i = 0
        while any(at[s] < len(seqs[s]) for s in range(2)):
            parts = []
            for s in range(2):
                n = min(sizes[(i + s) % len(sizes)], len(seqs[s]) - at[s])
                if n > 0 and not (s == 1 and i % 3 == 1):                           # sequence 1 sits out some steps
                    parts.append((s, n))
            i += 1
            if not parts:
                continue
            rows = torch.cat([seqs[s][at[s]:at[s] + n] for s, n in parts])
            src = rows.to(device) if norm else rows.to(dt).to(device)
            q_start = torch.tensor(np.cumsum([0] + [n for _, n in parts]), dtype=torch.int32, device=device)
            kv_len = torch.tensor([at[s] + n for s, n in parts], dtype=torch.int32, device=device)
            ss = torch.tensor([slots[s] for s, _ in parts], dtype=torch.int32, device=device)
            phase = torch.tensor([steps[s] & 1 for s, _ in parts], dtype=torch.int32, device=device)
            out32 = torch.empty(len(rows), C, dtype=torch.float32, device=device)
            out = torch.empty(len(rows), C, dtype=dt, device=device)
            ops.causal_conv(src, w.to(device), state, q_start, kv_len, ss, phase, len(parts), out=out, out32=out32,
                            norm_weight=nw.to(device) if norm else None, eps=1e-5,
                            bias=bias.to(device) if bias is not None else None, identity=1.0 if norm else 0.0)
            row = 0
            for s, n in parts:
                got[s].append(out32[row:row + n].cpu())
                assert torch.allclose(out[row:row + n].float().cpu(), out32[row:row + n].to(dt).float().cpu())
                row += n
                at[s] += n
                steps[s] += 1
        for s in range(2):
            assert torch.allclose(torch.cat(got[s]).double(), want[s], atol=2e-5, rtol=2e-5)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("taps,norm", [(4, True), (3, False), (1, True), (8, False), (2, True)])
def test_causal_conv_of_many_rows(device, dtype, taps, norm):
    """A step of 640 rows (the kernel that walks tiles of rows): a sequence that starts in it, one that goes on from
    its state (whose first tokens come mid-tile), one of two tokens, one of one token that began steps ago."""
    from tessweave_engine_amd.kernels import ops
    g = torch.Generator().manual_seed(taps + 10 * norm)
    C, dt = 48, tdtype(dtype)
    w = torch.randn(C, taps, generator=g)
    bias = None if norm else torch.randn(C, generator=g)
    nw = 1 + 0.3 * torch.randn(C, generator=g)
    lengths, before = [300, 331, 2, 7], [0, 5, 0, 6]              # tokens in all, of which in an earlier step
    seqs = [torch.randn(n, C, generator=g) for n in lengths]
    if not norm:
        seqs = [s.to(dt).float() for s in seqs]
    want = []
    for s in seqs:
        v = plain.rms_norm(s.double(), nw.double(), 1e-5) if norm else s.double()
        want.append((v if norm else 0) + plain.causal_conv(v, w.double()) + (0 if norm else bias.double()))
    state = torch.zeros(4, 2, max(taps - 1, 1), C, device=device)
    slots = torch.tensor([3, 1, 0, 2], dtype=torch.int32, device=device)

    def step(parts, phases):
        rows = torch.cat([seqs[s][lo:hi] for s, lo, hi in parts])
        src = rows.to(device) if norm else rows.to(dt).to(device)
        q_start = torch.tensor(np.cumsum([0] + [hi - lo for _, lo, hi in parts]), dtype=torch.int32, device=device)
        kv_len = torch.tensor([hi for _, _, hi in parts], dtype=torch.int32, device=device)
        out32 = torch.empty(len(rows), C, device=device)
        out = torch.empty(len(rows), C, dtype=dt, device=device)
        scratch = torch.empty(len(rows), device=device)
        ops.causal_conv(src, w.to(device), state, q_start, kv_len, slots[[s for s, _, _ in parts]].contiguous(),
                        torch.tensor(phases, dtype=torch.int32, device=device), len(parts), out=out, out32=out32,
                        norm_weight=nw.to(device) if norm else None, eps=1e-5, bias=bias.to(device) if bias is not None else None,
                        identity=1.0 if norm else 0.0, row_scratch=scratch)
        assert torch.allclose(out.float().cpu(), out32.to(dt).float().cpu())
        return out32.cpu()

    step([(1, 0, 5), (3, 0, 6)], [0, 0])                              # the earlier step of sequences 1 and 3
    got = step([(0, 0, 300), (1, 5, 331), (2, 0, 2), (3, 6, 7)], [0, 1, 0, 1])
    at = 0
    for s, lo, hi in [(0, 0, 300), (1, 5, 331), (2, 0, 2), (3, 6, 7)]:
        assert torch.allclose(got[at:at + hi - lo].double(), want[s][lo:hi], atol=2e-5, rtol=2e-5), s
        at += hi - lo
    # and the state it left: one more token of sequence 1 from a short step
    extra = torch.randn(1, C, generator=g)
    if not norm:
        extra = extra.to(dt).float()
    seqs[1] = torch.cat([seqs[1], extra])
    v = plain.rms_norm(seqs[1].double(), nw.double(), 1e-5) if norm else seqs[1].double()
    full = (v if norm else 0) + plain.causal_conv(v, w.double()) + (0 if norm else bias.double())
    got = step([(1, 331, 332)], [0])
    assert torch.allclose(got.double(), full[331:332], atol=2e-5, rtol=2e-5)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_gated_recurrence_carries_its_state(device, dtype):
    from tessweave_engine_amd.kernels import ops
    g = torch.Generator().manual_seed(5)
    R, blocks, T, dt = 24, 3, 400, tdtype(dtype)
    bs = R // blocks
    u = torch.randn(T, R, generator=g)
    ga, gi = torch.randn(T, R, generator=g) * 2, torch.randn(T, R, generator=g) * 2
    branch = torch.randn(T, R, generator=g).to(dt).float()
    lam = torch.randn(R, generator=g) * 2
    S = plain.gated_recurrence(u.double(), torch.sigmoid(ga.double()), torch.sigmoid(gi.double()), lam.double())
    want = 0.7 * S * plain.gelu_tanh(branch.double())
    # block b's recurrence gates, then its input gates
    gates = torch.cat([torch.cat([ga[:, b * bs:(b + 1) * bs], gi[:, b * bs:(b + 1) * bs]], 1) for b in range(blocks)], 1)
    state = torch.zeros(2, R, device=device)
    state[0] = float("nan")                                # another request's slot
    got, at = [], 0
    for n in (1, 5, 2, 1, 17, 14, 32, 33, 64, 200, 31):      # portions of one chunk, of exactly one, and of several
        out = torch.full((n, R + 3), float("nan"), dtype=dt, device=device)
        floats = ops.gated_recurrence_workspace_floats(1, n, R)
        assert (floats > 0) == (n > 32)
        ws = torch.full((max(floats, 1),), float("nan"), device=device)
        ops.gated_recurrence(gates[at:at + n].contiguous().to(device), u[at:at + n].contiguous().to(device),
                             branch[at:at + n].to(dt).to(device), lam.to(device), state,
                             torch.tensor([0, n], dtype=torch.int32, device=device),
                             torch.tensor([1], dtype=torch.int32, device=device), 1, n, out, blocks, 8.0, out_scale=0.7,
                             out_pad=3, workspace=ws)
        assert (out[:, R:] == 0).all()
        got.append(out[:, :R].float().cpu())
        at += n
    tol = 1e-5 if dtype == "float32" else 1e-2
    assert torch.allclose(torch.cat(got).double(), want, atol=tol, rtol=tol)
    assert torch.allclose(state[1].cpu().double(), S[-1], atol=1e-5, rtol=1e-5)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("n,blocks,n_in,n_out", [(1, 3, 8, 16), (37, 2, 40, 80), (130, 16, 128, 256)])
def test_block_diagonal_product(device, dtype, n, blocks, n_in, n_out):
    from tessweave_engine_amd.kernels import ops
    g = torch.Generator().manual_seed(n)
    dt = tdtype(dtype)
    x = torch.randn(n, blocks * n_in, generator=g).to(dt)
    w = (torch.randn(blocks, n_out, n_in, generator=g) / math.sqrt(n_in)).to(dt)
    bias = torch.randn(blocks * n_out, generator=g)
    want = plain.block_diagonal(x.double(), w.double(), bias.double().view(blocks, n_out))
    wide = torch.zeros(n, blocks * n_in + 8, dtype=dt, device=device)          # rows further apart than they are long
    wide[:, :blocks * n_in] = x.to(device)
    out = torch.empty(n, blocks * n_out, device=device)
    assert ops.can_block_diagonal(wide[:, :blocks * n_in], w.to(device))
    ops.block_diagonal(wide[:, :blocks * n_in], w.to(device), bias.to(device), out)
    tol = 2e-5 if dtype == "float32" else 2e-2
    assert torch.allclose(out.cpu().double(), want, atol=tol, rtol=tol)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("rows", [3, 40, 300])
def test_gated_product_with_gelu_and_a_factor(device, dtype, rows):
    """The matrix kernels' gated epilogue with the tanh form of gelu (few rows, 17-64 rows, tiled) and shuffled weights."""
    from tessweave_engine_amd.kernels import ops
    g = torch.Generator().manual_seed(rows)
    dt = tdtype(dtype)
    k, inter = 96, 160
    x = torch.randn(rows, k, generator=g).to(dt)
    gate = (torch.randn(inter, k, generator=g) / math.sqrt(k)).to(dt)
    up = (torch.randn(inter, k, generator=g) / math.sqrt(k)).to(dt)
    want = 0.7 * plain.gelu_tanh(x.double() @ gate.double().T) * (x.double() @ up.double().T)
    packed = ops.shuffle_weight(ops.interleave_glu_rows(gate.to(device), up.to(device)))
    out = torch.empty(rows, inter, dtype=dt, device=device)
    ops.linear_glu(x.to(device), packed, out, activation="gelu_tanh", factor=0.7)
    tol = 2e-5 if dtype == "float32" else 2e-2
    assert torch.allclose(out.cpu().double(), want, atol=tol, rtol=tol)


def test_small_kernels(device):
    from tessweave_engine_amd.kernels import ops
    g = torch.Generator().manual_seed(9)
    n, C, L = 5, 24, 3
    x = torch.randn(n, C, generator=g)
    y = torch.randn(n, C, generator=g)
    w = torch.randn(C, generator=g)
    hist = torch.randn(L + 1, 8, C, generator=g)
    mix = torch.randn(L + 1, generator=g)
    xd, hd = x.to(device), hist.to(device)
    ops.layer_end(xd, L - 1, branch=y.to(device), branch_weight=w.to(device), eps=1e-5, mult=0.4, history=hd, mix=mix.to(device))
    result = x.double() + 0.4 * plain.rms_unit(y.double(), 1e-5) * w.double()
    mixed = sum(mix[j].double() * hist[j, :n].double() for j in range(L)) + mix[L].double() * result
    assert torch.allclose(hd[L, :n].cpu().double(), result, atol=1e-5)
    assert torch.allclose(xd.cpu().double(), mixed, atol=1e-5)
    gu = torch.randn(n, 2 * C, generator=g)
    out = torch.empty(n, C, device=device)
    ops.gelu_mul(gu.to(device), out, 0.3)
    assert torch.allclose(out.cpu().double(), 0.3 * plain.gelu_tanh(gu[:, :C].double()) * gu[:, C:].double(), atol=1e-6)
    table = torch.randn(7, 2 * C, generator=g)
    ids = torch.tensor([3, -2, 0, 6, -1], dtype=torch.int32)
    feed = torch.tensor([5, 1], dtype=torch.int32)
    pre = torch.randn(n, 6, generator=g)
    out = torch.empty(n, 6, device=device)
    ops.token_gate(pre.to(device), table.to(device), ids.to(device), 12, out, feed=feed.to(device))
    real = torch.tensor([3, 1, 0, 6, 5])
    assert torch.allclose(out.cpu().double(), plain.gelu_tanh(pre.double()) * table[real, 12:18].double(), atol=1e-6)
    pos = torch.randn(9, C, generator=g)
    copy = torch.empty(n, C, device=device)
    xd = x.to(device)
    ops.add_table_rows(xd, pos.to(device), torch.tensor([4, 5, 6, 0, 8], dtype=torch.int32, device=device), copy=copy)
    assert torch.equal(xd.cpu(), x + pos[[4, 5, 6, 0, 8]]) and torch.equal(copy, xd)


# ---------------------------------------------------------------------------------------------------------
# whole models
# ---------------------------------------------------------------------------------------------------------

LENGTHS = {"odd": [61, 3, 40, 1, 29, 75], "wide": [50, 37, 2, 66], "one": [44, 9, 30]}


@pytest.fixture(scope="module", params=list(CONFIGS))
def model(request, tmp_path_factory, device):
    name = request.param
    c = CONFIGS[name]
    weights = make_weights(c, seed=len(name))
    folder = write_folder(tmp_path_factory.mktemp("kanavik_" + name), c, weights)
    g = torch.Generator().manual_seed(50 + len(name))
    tokens = {f"r{i}": torch.randint(0, c["vocab"], (n,), generator=g).tolist() for i, n in enumerate(LENGTHS[name])}
    want = {rid: plain.forward(c, weights, toks).numpy() for rid, toks in tokens.items()}
    return dict(name=name, config=c, weights=weights, folder=folder, tokens=tokens, want=want)


def check_all(model, got, dtype, only=None):
    for rid, want in model["want"].items():
        if only is not None and rid not in only:
            continue
        err = row_error(got[rid], want)
        assert np.isfinite(got[rid]).all()
        assert err.max() < BAR[dtype], (rid, int(err.argmax()), float(err.max()))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole_prompts(model, dtype):
    d = Driver(model["folder"], dtype, pages=24, page_size=8)
    got = d.run([[(rid, len(toks))] for rid, toks in model["tokens"].items()], model["tokens"])
    check_all(model, got, dtype)
    d.close()


@pytest.mark.parametrize("dtype,graphs", [("float32", True), ("float32", False), ("bfloat16", True)])
def test_token_by_token(model, dtype, graphs):
    """Every token decoded alone from the first on (the first tokens of a sequence included)."""
    rid = "r0"
    d = Driver(model["folder"], dtype, pages=24, page_size=4, graphs=graphs)
    got = d.run([[(rid, 1)] for _ in model["tokens"][rid]], model["tokens"])
    check_all(model, got, dtype, only=[rid])
    if graphs:
        assert d.stepper.graph_replays > 0
    d.close()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("sizes", [[2], [3, 1, 2], [16, 5, 2, 2, 9], [7, 8, 1]])
def test_portions(model, dtype, sizes):
    rid = max(model["tokens"], key=lambda r: len(model["tokens"][r]))
    total, schedule, i = len(model["tokens"][rid]), [], 0
    while total:
        n = min(sizes[i % len(sizes)], total)
        schedule.append([(rid, n)])
        total -= n
        i += 1
    d = Driver(model["folder"], dtype, pages=40, page_size=4)
    got = d.run(schedule, model["tokens"])
    check_all(model, got, dtype, only=[rid])
    d.close()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", [0, 1])
def test_unequal_batches_few_pages_two_slots(model, dtype, seed):
    """Portions of some requests beside single tokens of others; at most two requests live, so that every
    state slot is used again, and a page pool that only just holds them."""
    import random
    rng = random.Random(seed)
    tokens = model["tokens"]
    pending, live, schedule = list(tokens), {}, []
    while pending or live:
        while pending and len(live) < 2:
            rid = pending.pop(0)
            live[rid] = dict(left=len(tokens[rid]), prompt=rng.randrange(1, len(tokens[rid]) + 1))
        parts = []
        for rid, r in list(live.items()):
            if len(live) > 1 and rng.random() < 0.25:
                continue
            n = min(r["left"], rng.choice([2, 3, 5, 11, 16]) if r["prompt"] > 0 else 1)
            r["prompt"] -= n
            r["left"] -= n
            parts.append((rid, n))
            if r["left"] == 0:
                del live[rid]
        if parts:
            schedule.append(parts)
    page = 8
    longest = sorted(len(t) for t in tokens.values())[-2:]
    pages = sum((n + page - 1) // page for n in longest)
    d = Driver(model["folder"], dtype, pages=pages, page_size=page, max_requests=2)
    got = d.run(schedule, tokens)
    check_all(model, got, dtype)
    d.close()


def test_ways_of_cutting_agree(model):
    """float32: whole, token by token and in portions beside another request differ by rounding only."""
    tokens = model["tokens"]
    rid, other = "r0", "r2"
    runs = []
    for schedule in ([[(rid, len(tokens[rid]))]],
                     [[(rid, 1)] for _ in tokens[rid]],
                     [[(other, 1), (rid, 5)]] + [[(rid, 2), (other, 1)] for _ in range(500)]):
        d = Driver(model["folder"], "float32", pages=40, page_size=4)
        fixed, used = [], {}
        for parts in schedule:
            parts = [(r, min(n, len(tokens[r]) - used.get(r, 0))) for r, n in parts]
            parts = [(r, n) for r, n in parts if n > 0]
            for r, n in parts:
                used[r] = used.get(r, 0) + n
            if parts:
                fixed.append(parts)
        runs.append(d.run(fixed, tokens)[rid])
        d.close()
    for other_run in runs[1:]:
        assert row_error(other_run, runs[0]).max() < 2e-5


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_prompt_in_one_step_then_portions(device, tmp_path, dtype):
    """600 tokens: 520 in one step (the kernels' forms for many rows: norm statistics formed once, the recurrence
    in chunks, attention over many tiles), then portions of 64, 15 and 1."""
    c = CONFIGS["odd"]
    weights = make_weights(c, seed=13)
    folder = write_folder(tmp_path, c, weights)
    toks = torch.randint(0, c["vocab"], (600,), generator=torch.Generator().manual_seed(4)).tolist()
    want = plain.forward(c, weights, toks).numpy()
    d = Driver(folder, dtype, pages=80, page_size=8)
    got = d.run([[("a", 520)], [("a", 64)], [("a", 15)], [("a", 1)]], {"a": toks})["a"]
    err = row_error(got, want)
    assert err.max() < BAR[dtype], (int(err.argmax()), float(err.max()))
    d.close()


def test_long_decoding_past_every_window(device, tmp_path):
    """400 tokens decoded one by one from graphs after a short prompt: the windows (7, 33) pass over decoded
    tokens, pages leave the windowed groups and are taken again."""
    c = CONFIGS["odd"]
    weights = make_weights(c, seed=11)
    folder = write_folder(tmp_path, c, weights)
    toks = torch.randint(0, c["vocab"], (420,), generator=torch.Generator().manual_seed(3)).tolist()
    want = plain.forward(c, weights, toks).numpy()
    d = Driver(folder, "float32", pages=70, page_size=16)
    got = d.run([[("a", 20)]] + [[("a", 1)] for _ in range(400)], {"a": toks})["a"]
    err = row_error(got, want)
    assert err.max() < BAR["float32"], (int(err.argmax()), float(err.max()))
    assert d.stepper.graph_replays > 300
    d.close()


@pytest.mark.parametrize("name", ["odd", "wide"])
def test_greedy_generation_through_the_scheduler(device, tmp_path, name):
    """`engine_for(...).generate`: the package's entry point, scheduler, sampler and lookahead. Every generated
    token must be the plain implementation's best token for the text so far (checked where its lead is clear)."""
    from tessweave_engine_amd.cli import engine_for
    c = CONFIGS[name]
    weights = make_weights(c, seed=21)
    folder = write_folder(tmp_path, c, weights)
    g = torch.Generator().manual_seed(8)
    prompts = [torch.randint(0, c["vocab"], (n,), generator=g).tolist() for n in (5, 23, 1, 40, 12, 30)]
    engine = engine_for(folder, dtype="float32", max_context=128, kv_blocks=40, block_size=8, max_active=3,
                        prefill_chunk=16, no_prefix_cache=False)
    try:
        outputs = engine.generate(prompts, max_tokens=24, temperature=0.0)
    finally:
        engine.close()
    clear = 0
    for prompt, out in zip(prompts, outputs):
        assert len(out) == 24
        logits = plain.forward(c, weights, prompt + out)[len(prompt) - 1:-1]
        top = logits.topk(2, -1)
        for t, token in enumerate(out):
            if top.values[t, 0] - top.values[t, 1] > 1e-3:
                assert token == int(top.indices[t, 0]), (t, token)
                clear += 1
    assert clear > 100

"""The Dinutar design on the GPU against the plain implementation (`plain_dinutar.py`).

Mechanisms alone (each kernel against the plain function of the same mechanism: the hashed pair embedding with its
carried token, the norm after the sum with and without pending partial sums, the stretched rotary tables, the
per-head matrices, retention over portions with carried state in reused slots, the unit norm with its gate), then
whole models through the package's loader, cache manager and step function: prefill against token-by-token
decoding, portions down to two tokens, unequal batches against each request alone, few pages and slots that are
freed and used again, attention made sharp so that single keys far back carry the result, long decoding from HIP
graphs, and greedy generation through the scheduler.

Bars: float32 rows must agree with the float64 plain implementation to 2e-5 of the logits' spread (the kernels sum
in other orders); bfloat16 to 3 % of it (bfloat16 rounds to 0.4 %, a few dozen roundings deep). A unit norm behind a
sum of products that nearly cancel magnifies its inputs' rounding, so in bfloat16 one row in fifty may lie up to
twice as far.
"""
import math

import numpy as np
import pytest
import torch

import plain_dinutar as plain
from dinutar_util import CONFIGS, Driver, make_weights, row_error, write_folder

pytestmark = pytest.mark.gpu

BAR = {"float32": 2e-5, "bfloat16": 3e-2}


def tdtype(name):
    return getattr(torch, name)


def ints(values, device):
    return torch.tensor(values, dtype=torch.int32, device=device)


# ---------------------------------------------------------------------------------------------------------
# mechanisms alone
# ---------------------------------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_hashed_pair_embedding_carries_the_last_token(device, dtype):
    """Three sequences in one launch: one at its start (its first token takes the table's last row), one that goes on
    with several tokens, one that goes on with a single fed token; stale state in the copies that must not be read."""
    from tessweave_engine_amd.kernels import ops
    dt = tdtype(dtype)
    g = torch.Generator().manual_seed(0)
    V, C, B, mp, mc, scale, eps = 50, 72, 13, 1000003, 7, 1.3, 1e-5
    table = torch.randn(V, C, generator=g).to(dt)
    pairs = torch.randn(B + 1, C, generator=g).to(dt)
    w = 1 + 0.3 * torch.randn(C, generator=g)
    seqs = {"a": [3, 49, 49, 0, 7], "b": [11, 12, 13, 14, 15, 16], "c": [20, 21, 22]}
    want = {k: plain.embed(v, table.double(), pairs.double(), scale, B, mp, mc, w.double(), eps) for k, v in seqs.items()}
    # this step: all of a, b's tokens 2.., c's last token (which comes through the feed)
    ids = ints(seqs["a"] + seqs["b"][2:] + [-2], device)
    feed = ints([5, seqs["c"][2]], device)
    q_start, kv_len = ints([0, 5, 9, 10], device), ints([5, 6, 3], device)
    slots, phase = ints([2, 0, 1], device), ints([0, 1, 0], device)
    state = torch.full((3, 2), 40, dtype=torch.int32, device=device)          # stale values everywhere
    state[0, 1] = seqs["b"][1]
    state[1, 0] = seqs["c"][1]
    x = torch.empty(10, C, dtype=torch.float32, device=device)
    out = torch.empty(10, C, dtype=dt, device=device)
    ops.embed_hashed(ids, table.to(device), pairs.to(device), w.to(device), q_start, kv_len, slots, phase, state, 3, B, mp, mc,
                     scale, eps, x, out=out, feed=feed)
    full = torch.cat([want["a"], want["b"][2:], want["c"][2:]]).float()
    assert torch.allclose(x.cpu(), full, atol=1e-5)
    assert torch.equal(out.cpu(), x.cpu().to(dt))
    assert state.cpu().tolist() == [[seqs["b"][-1], seqs["b"][1]], [seqs["c"][1], seqs["c"][2]], [40, seqs["a"][-1]]]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("n,hidden,splits", [(5, 96, 0), (3, 90, 3), (70, 4104, 2), (2, 9000, 0), (4, 20000, 1)])
def test_norm_after_the_sum(device, dtype, n, hidden, splits):
    from tessweave_engine_amd.kernels import ops
    g = torch.Generator().manual_seed(hidden)
    x = torch.randn(n, hidden, generator=g)
    y = torch.randn(max(splits, 1), n, hidden, generator=g)
    scale, w = torch.randn(hidden, generator=g), 1 + 0.2 * torch.randn(hidden, generator=g)
    alpha, eps = 1.7, 1e-5
    want = plain.rms_norm(alpha * x.double() + scale.double() * y.double().sum(0), w.double(), eps)
    xd = x.to(device)
    out = torch.empty(n, hidden, dtype=tdtype(dtype), device=device)
    if splits:
        ops.residual_norm(xd, w.to(device), eps, out=out, add=y.to(device), scale=scale.to(device), alpha=alpha)
    else:
        wide = torch.zeros(n, hidden + 8, device=device)
        wide[:, :hidden] = y[0].to(device)
        ops.residual_norm(xd, w.to(device), eps, out=out, y=wide[:, :hidden], scale=scale.to(device), alpha=alpha)
    assert torch.allclose(xd.cpu().double(), want, atol=2e-5, rtol=1e-5)
    assert torch.equal(out.cpu(), xd.cpu().to(tdtype(dtype)))
    # no sublayer result at all, no scale: the norm of alpha x
    x2 = x.to(device)
    ops.residual_norm(x2, w.to(device), eps, alpha=alpha)
    assert torch.allclose(x2.cpu().double(), plain.rms_norm(alpha * x.double(), w.double(), eps), atol=2e-5, rtol=1e-5)


def test_stretched_rotary_tables(device):
    from tessweave_engine_amd.kernels import ops
    from tessweave_engine_amd.parts import RotaryEmbedding
    for dims, base, stretch in [(16, 1e4, (2.0, 64, 8.0, 1.0)), (8, 100.0, (4.0, 24, 6.0, 0.5)), (64, 1e6, None),
                                (4, 20.0, (8.0, 8, 2.0, 1.0))]:
        part = RotaryEmbedding(dims, base, dims, stretch=stretch)
        scaling = dict(zip(("factor", "original", "fast", "slow"), stretch)) if stretch else None
        f, mag = plain.rotary_frequencies(dims, base, scaling)
        assert torch.allclose(part.frequencies().double(), f, rtol=1e-6)
        assert part.magnitude == pytest.approx(mag)
        part.bind({}, torch.float32, device)
        pos = ints([0, 1, 5, 300, 4097], device)
        cos = torch.empty(5, dims // 2, device=device)
        sin = torch.empty(5, dims // 2, device=device)
        ops.rope_table(pos, part.inv_freq, cos, sin, part.magnitude)
        angle = pos.cpu().double().view(-1, 1) * f
        assert torch.allclose(cos.cpu().double(), torch.cos(angle) * mag, atol=3e-4)
        assert torch.allclose(sin.cpu().double(), torch.sin(angle) * mag, atol=3e-4)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("n,heads,n_in,n_out", [(1, 3, 24, 48), (37, 5, 16, 80), (100, 1, 96, 8), (18, 12, 128, 132)])
def test_head_linear(device, dtype, n, heads, n_in, n_out):
    """One matrix per head over heads that lie side by side with gaps between them, into rows with gaps."""
    from tessweave_engine_amd.kernels import ops
    dt = tdtype(dtype)
    g = torch.Generator().manual_seed(n)
    sx, so = n_in + 8, n_out + 16
    x = torch.randn(n, heads * sx + 8, generator=g).to(dt)
    w = (torch.randn(heads, n_out, n_in, generator=g) / math.sqrt(n_in)).to(dt)
    out = torch.full((n, heads * so), 7.0, dtype=dt, device=device)
    ops.head_linear(x.to(device), sx, w.to(device), out, so)
    got = out.cpu().view(n, heads, so)
    want = torch.einsum("nai,aoi->nao", x[:, :heads * sx].view(n, heads, sx)[..., :n_in].double(), w.double())
    assert torch.allclose(got[..., :n_out].double(), want, atol=2e-2 if dtype == "bfloat16" else 1e-5)
    assert (got[..., n_out:] == 7.0).all()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H,L,R,page,lengths,splits", [
    (5, 48, 16, 4, [1, 7, 70], 1),             # fewer heads than a tile, pages of four keys, one key only
    (20, 96, 32, 16, [300, 17, 1000], 0),      # two tiles of heads, key ranges as the launcher would choose them
    (16, 192, 64, 16, [2049, 33], 9),          # ranges that get no key at all for the short sequence
    (1, 16, 16, 8, [129], 3),
])
def test_one_token_attention_over_the_cached_latent(device, dtype, H, L, R, page, lengths, splits):
    """All heads of a sequence against its one cached head: key rows [c | kr] on pages handed out in reverse order,
    values = c once more, transposed inside a page; one key far back carries most of a head's weight; what lies in a
    page behind a sequence's end is NaN and must not reach a sum."""
    from tessweave_engine_amd.kernels import ops
    dt = tdtype(dtype)
    g = torch.Generator().manual_seed(L + R)
    K, scale = L + R, 0.3
    blocks = [(n + page - 1) // page for n in lengths]
    n_pages = sum(blocks)
    keys = torch.full((n_pages + 1, 1, page, K), float("nan"), dtype=dt)
    values = torch.full((n_pages + 1, 1, L, page), float("nan"), dtype=dt)
    table = torch.full((len(lengths), max(blocks)), -1, dtype=torch.int32)
    q = (torch.randn(len(lengths), H, K, generator=g)).to(dt)
    want, free = [], list(range(n_pages, 0, -1))
    for s, n in enumerate(lengths):
        rows = torch.randn(n, K, generator=g).to(dt)
        far = n // 5
        rows[far] = (q[s, 0].float() * 0.5).to(dt)                 # head 0 of this sequence looks at this key above all
        for b in range(blocks[s]):
            pg = free.pop(0)
            table[s, b] = pg
            part = rows[b * page:(b + 1) * page]
            keys[pg, 0, :len(part)] = part
            values[pg, 0, :, :len(part)] = part[:, :L].T
        sc = torch.einsum("hk,nk->hn", q[s].double(), rows.double()) * scale
        want.append(torch.softmax(sc, -1) @ rows[:, :L].double())
    n_seqs = len(lengths)
    if splits == 0:
        splits = ops.latent_decode_splits(n_seqs, H, max(lengths))
    floats = ops.latent_decode_workspace_floats(n_seqs, H, L, splits)
    ws = torch.full((max(floats, 1),), float("nan"), device=device)
    out = torch.zeros(n_seqs, H * L, dtype=dt, device=device)
    ops.latent_decode(q.view(n_seqs, H * K).to(device), keys.to(device), values.to(device), table.to(device),
                      ints(list(range(n_seqs + 1)), device), ints(lengths, device), n_seqs, out, H, scale, splits=splits,
                      workspace=ws if floats else None)
    got = out.cpu().double().view(n_seqs, H, L)
    for s in range(n_seqs):
        err = (got[s] - want[s]).abs().max().item()
        assert err < (3e-2 if dtype == "bfloat16" else 2e-5), (s, err)


def retention_case(H, D, E, rot_dims, decay, lengths, seed):
    """Raw projections [T, 2 H D + 2 H E] of several sequences and what the mechanism gives for each (float64)."""
    g = torch.Generator().manual_seed(seed)
    width = 2 * H * D + 2 * H * E
    rot = {"dims": rot_dims, "base": 30.0} if rot_dims else None
    eye = torch.eye(width, dtype=torch.float64)
    raws, wants = [], []
    for T in lengths:
        raw = torch.randn(T, width, generator=g).to(torch.bfloat16)
        cols = [0, H * D, 2 * H * D, 2 * H * D + H * E, width]
        sel = [eye[cols[i]:cols[i + 1]] for i in range(4)]
        wants.append(plain.retention(raw.double(), sel[0], sel[1], sel[2], sel[3], torch.eye(H * E, dtype=torch.float64), H, D, E,
                                     decay, 1e-5, torch.arange(T), rot))
        raws.append(raw)
    return raws, wants, rot


@pytest.mark.parametrize("chunked", [True, False])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H,D,E,rot_dims,decay,cuts", [
    (2, 16, 16, 16, [0.5, 1.0], [[5, 1, 1, 30], [1, 36]]),                 # a decay of exactly one
    (3, 48, 80, 16, [0.9, 0.99, 0.999], [[70, 2, 3], [40, 35], [1] * 6]),  # values in two column slices, partial rotation
    (1, 128, 32, 0, [0.97], [[17, 130], [147]]),                            # no rotation, portions longer than any chunk
    (4, 32, 144, 32, [0.8, 0.9, 0.95, 0.995], [[200, 1, 1], [64, 64, 74]]),
    (1, 256, 48, 64, [0.999], [[33, 31, 70]]),                              # the longest keys: chunks of 32
    (2, 64, 64, 64, [0.99, 0.9999], [[1500, 3, 300], [5, 700, 1098]]),      # long portions: several segments a sequence
    (1, 128, 16, 32, [0.995], [[2304]]),
])
def test_retention_over_portions(device, dtype, H, D, E, rot_dims, decay, cuts, chunked):
    """Sequences cut differently run side by side, step after step, from state slots that held other values; the
    per-head unit norm and the gate follow. Both kernels: the one that walks chunks on the matrix unit and the one
    that walks token by token. Heads are padded on the device only in the model; here sizes are multiples of 16."""
    from tessweave_engine_amd.kernels import ops
    dt = tdtype(dtype)
    lengths = [sum(c) for c in cuts]
    raws, wants, rot = retention_case(H, D, E, rot_dims, decay, lengths, seed=D + E)
    state = torch.randn(len(cuts) + 1, H, D, E, device=device)                # stale
    slots = list(range(len(cuts), 0, -1))
    for s in slots:
        state[s].zero_()                                                    # what opening a request does
    dec = torch.tensor(decay, dtype=torch.float32, device=device)
    f = plain.rotary_frequencies(rot_dims, 30.0)[0].float().to(device) if rot_dims else None
    at = [0] * len(cuts)
    got = [torch.zeros(n, H * E) for n in lengths]
    for step in range(max(len(c) for c in cuts)):
        live = [i for i, c in enumerate(cuts) if step < len(c)]
        rows = torch.cat([raws[i][at[i]:at[i] + cuts[i][step]] for i in live]).to(dt).to(device)
        counts = [cuts[i][step] for i in live]
        q_start = ints(np.concatenate([[0], np.cumsum(counts)]).tolist(), device)
        pos = ints([p for i in live for p in range(at[i], at[i] + cuts[i][step])], device)
        cos = sin = None
        if rot_dims:
            cos = torch.empty(rows.shape[0], rot_dims // 2, device=device)
            sin = torch.empty_like(cos)
            ops.rope_table(pos, f, cos, sin)
        o = torch.empty(rows.shape[0], H * E, device=device)
        longest = max(counts) if chunked else 0
        floats = ops.retention_workspace_floats(len(live), longest, H, D, E) if chunked else 0
        ws = torch.full((floats,), float("nan"), device=device) if floats else None
        ops.retention(rows, 0, H * D, 2 * H * D, cos, sin, dec, state, q_start, ints([slots[i] for i in live], device),
                      0, len(live), o, D ** -0.5, max_q_len=longest, workspace=ws)
        act = torch.empty(rows.shape[0], H * E, dtype=dt, device=device)
        ops.unit_gate(o, rows[:, 2 * H * D + H * E:], act, H, E, E, 1e-5)
        row = 0
        for i, n in zip(live, counts):
            got[i][at[i]:at[i] + n] = act[row:row + n].float().cpu()
            at[i] += n
            row += n
    for i in range(len(cuts)):
        err = (got[i].double() - wants[i]).abs().max().item()
        assert err < (4e-2 if dtype == "bfloat16" else 5e-4), (i, err)      # (sums over up to 2,300 tokens at decays near one)


def test_unit_gate_pads(device):
    """Heads laid out with tails: the mean runs over the real elements, the tails come out as zeros."""
    from tessweave_engine_amd.kernels import ops
    H, E, Ep, n = 3, 20, 32, 9
    o = torch.zeros(n, H, Ep)
    o[..., :E] = torch.randn(n, H, E)
    gate = torch.randn(n, H, Ep)
    out = torch.full((n, H * Ep), 5.0, device=device)
    ops.unit_gate(o.view(n, -1).to(device), gate.view(n, -1).to(device), out, H, E, Ep, 1e-6)
    want = plain.rms_unit(o[..., :E].double(), 1e-6) * torch.nn.functional.silu(gate[..., :E].double())
    got = out.cpu().view(n, H, Ep)
    assert torch.allclose(got[..., :E].double(), want, atol=1e-5) and (got[..., E:] == 0).all()


def test_relu_squared_in_place(device):
    from tessweave_engine_amd.kernels import ops
    x = torch.randn(7, 40).to(torch.bfloat16)
    buf = torch.zeros(7, 48, dtype=torch.bfloat16, device=device)
    buf[:, :40] = x.to(device)
    ops.relu_squared(buf[:, :40])
    assert torch.equal(buf[:, :40].cpu(), (torch.relu(x.float()) ** 2).to(torch.bfloat16)) and (buf[:, 40:] == 0).all()
    parts = torch.randn(3, 7, 40)
    ops.relu_squared(buf[:, :40], partial=parts.to(device))
    assert torch.equal(buf[:, :40].cpu(), (torch.relu(parts[0] + parts[1] + parts[2]) ** 2).to(torch.bfloat16)) and (buf[:, 40:] == 0).all()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("m,n,k,shuffled", [(65, 40, 96, True), (300, 272, 64, False), (2048, 1408, 512, True), (130, 4096, 2048, True)])
def test_product_with_relu_squared_in_its_epilogue(device, dtype, m, n, k, shuffled):
    """Against the product followed by the activation's own kernel (the same sums; one rounding instead of two), with
    and without split-K sums, with a bias."""
    from tessweave_engine_amd.kernels import ops
    dt = tdtype(dtype)
    g = torch.Generator().manual_seed(m + n)
    x = torch.randn(m, k, generator=g).to(dt).to(device)
    w = (torch.randn(n, k, generator=g) / math.sqrt(k)).to(dt).to(device)
    bias = torch.randn(n, generator=g).to(device)
    weight = ops.shuffle_weight(w) if shuffled else w
    floats = ops.linear_workspace_bytes(dt, m, n, k) // 4
    ws = torch.empty(max(floats, 1), device=device)
    out = torch.empty(m, n, dtype=dt, device=device)
    ops.linear_act(x, weight, out, "relu_squared", bias=bias, workspace=ws if floats else None)
    want = torch.relu(x.double() @ w.double().T + bias.double()) ** 2
    tol = 3e-2 if dtype == "bfloat16" else 1e-4
    assert ((out.double() - want).abs() <= tol * (1 + want.abs())).all()


# ---------------------------------------------------------------------------------------------------------
# whole models
# ---------------------------------------------------------------------------------------------------------

LENGTHS = {"odd": [61, 3, 40, 1, 29, 75], "wide": [50, 37, 2, 66], "one": [44, 9, 30], "deep": [33, 5, 47]}


@pytest.fixture(scope="module", params=list(CONFIGS))
def model(request, tmp_path_factory, device):
    name = request.param
    c = CONFIGS[name]
    weights = make_weights(c, seed=len(name))
    folder = write_folder(tmp_path_factory.mktemp("dinutar_" + name), c, weights)
    g = torch.Generator().manual_seed(50 + len(name))
    tokens = {f"r{i}": torch.randint(0, c["vocab"], (n,), generator=g).tolist() for i, n in enumerate(LENGTHS[name])}
    want = {rid: plain.forward(c, weights, toks).numpy() for rid, toks in tokens.items()}
    return dict(name=name, config=c, weights=weights, folder=folder, tokens=tokens, want=want)


def check_rows(err, dtype, what=""):
    """ERR: one relative error per row (see the bars at the top)."""
    err = np.asarray(err)
    if dtype == "bfloat16":
        assert err.max() < 2 * BAR[dtype], (what, int(err.argmax()), float(err.max()))
        assert (err > BAR[dtype]).sum() <= max(1, len(err) // 50), (what, np.nonzero(err > BAR[dtype])[0].tolist())
    else:
        assert err.max() < BAR[dtype], (what, int(err.argmax()), float(err.max()))


def check_all(model, got, dtype, only=None):
    errs = []
    for rid, want in model["want"].items():
        if only is not None and rid not in only:
            continue
        assert np.isfinite(got[rid]).all()
        errs.append(row_error(got[rid], want))
    check_rows(np.concatenate(errs), dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole_prompts(model, dtype):
    d = Driver(model["folder"], dtype, pages=24, page_size=8)
    got = d.run([[(rid, len(toks))] for rid, toks in model["tokens"].items()], model["tokens"])
    check_all(model, got, dtype)
    d.close()


def test_stream_after_every_layer(model):
    """float32: the residual stream after each layer run against the plain implementation's."""
    from tessweave_engine_amd.engine.step import StepEntry
    rid = "r0"
    toks = model["tokens"][rid]
    want = []
    plain.forward(model["config"], model["weights"], toks, layers_out=want)
    d = Driver(model["folder"], "float32", pages=24, page_size=8, graphs=False)
    seq = d.cache.open(rid)
    ctx, ordered, _ = d.stepper.prepare([StepEntry(seq, list(toks), [len(toks) - 1])])
    seen = []
    ctx.segment_end = lambda i: seen.append(ctx.scratch("residual", (ctx.n_tokens, model["config"]["width"]), torch.float32).clone())
    with torch.cuda.stream(d.stepper.stream):
        d.stepper.upload(ctx)
        d.model.forward(ctx)
    d.stepper.synchronize()
    d.stepper.finish(ordered)
    assert len(seen) == len(want)
    for i, (got, ref) in enumerate(zip(seen, want)):
        assert torch.allclose(got.cpu().double(), ref, atol=5e-5), i
    d.close()


@pytest.mark.parametrize("dtype,graphs", [("float32", True), ("float32", False), ("bfloat16", True)])
def test_token_by_token(model, dtype, graphs):
    """Every token decoded alone from the first on (the first tokens of a sequence included)."""
    rid = "r0"
    d = Driver(model["folder"], dtype, pages=24, page_size=4, graphs=graphs)
    got = d.run([[(rid, 1)] for _ in model["tokens"][rid]], model["tokens"])
    check_all(model, got, dtype, only=[rid])
    if graphs and d.model.graph_safe_model:
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
    state slot is used again (retention states, last tokens), and a page pool that only just holds them."""
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
@pytest.mark.parametrize("name", ["odd", "wide"])
def test_sharp_attention_over_a_long_prompt(device, tmp_path, dtype, name):
    """Queries eight times as large: every softmax sits on one or two keys, wherever they lie among hundreds (far back,
    at a page's edge, the first token). 600 tokens: 330 in one step (many row tiles, retention over many chunks),
    then portions of 64, 15, 2 and single tokens, on pages of four tokens handed out in an order of their own.
    Such a softmax magnifies the rounding of its scores (two keys that nearly tie change places): float32 rows must
    agree to 1e-3, where a key that is lost or seen wrongly moves a row by a tenth and more; in bfloat16 the typical
    row must stay within the bar."""
    c = CONFIGS[name]
    # (bfloat16 rounds a score of 50 by 0.2, a fifth of a weight: its queries are three times as large, not eight)
    weights = make_weights(c, seed=13, sharp=8.0 if dtype == "float32" else 3.0)
    folder = write_folder(tmp_path, c, weights)
    toks = torch.randint(0, c["vocab"], (600,), generator=torch.Generator().manual_seed(4)).tolist()
    want = plain.forward(c, weights, toks).numpy()
    d = Driver(folder, dtype, pages=180, page_size=4, max_step_tokens=64)
    # take and give back pages first, so that the request's pages are not in order
    warm = {"w0": toks[:37], "w1": toks[:90]}
    d.step([("w0", 37), ("w1", 90)], warm)
    d.end("w0")
    schedule = [[("a", 330)], [("a", 64)], [("a", 15)], [("a", 2)]] + [[("a", 1)]] * 9 + [[("a", 90)], [("a", 90)]]
    got = d.run(schedule, {"a": toks})["a"]
    d.end("w1")
    err = row_error(got, want)
    if dtype == "float32":
        assert err.max() < 1e-3, (int(err.argmax()), float(err.max()))
    else:
        assert np.median(err) < BAR[dtype], float(np.median(err))
    d.close()


def random_config(seed):
    """A configuration drawn at random: layer kinds in any order, sizes that are mostly no multiples of 16, readers of
    earlier latents, stretched and plain rotations, layers with and without a feed-forward."""
    import random
    from dinutar_util import config, latent, retention
    rng = random.Random(seed)
    even = lambda lo, hi: 2 * rng.randint(lo // 2, hi // 2)
    layers, writers = [], []
    for i in range(rng.randint(2, 6)):
        ff = rng.choice([None, rng.randint(3, 20) * 8, rng.randint(20, 150)])
        scaling = rng.choice([None, (rng.choice([2.0, 4.0, 16.0]), rng.choice([8, 32, 100]), rng.choice([4.0, 32.0]), rng.choice([0.5, 1.0]))])
        if rng.random() < 0.55 or i == 0 and rng.random() < 0.5:
            if writers and rng.random() < 0.4:
                j = rng.choice(writers)
                m = layers[j]["mixer"]
                lay = latent(rng.randint(1, 19), even(2, 60), m["rot_dim"], rng.randint(1, 70), m["kv_rank"], rng.uniform(0.05, 0.4), kv_from=j, ff=ff)
                lay["mixer"]["rot"] = m["rot"]
            else:
                rot_dim = even(2, 40)
                lay = latent(rng.randint(1, 19), even(2, 60), rot_dim, rng.randint(1, 70), rng.randint(4, 150), rng.uniform(0.05, 0.4),
                             base=rng.choice([50.0, 1e4, 1e6]), scaling=scaling, ff=ff)
                writers.append(i)
        else:
            heads, dim = rng.randint(1, 5), even(2, 70)
            lay = retention(heads, dim, rng.randint(1, 150), [rng.choice([1.0, rng.uniform(0.3, 0.9999)]) for _ in range(heads)],
                            even(2, dim), base=rng.choice([30.0, 1e4]), scaling=scaling, ff=ff)
        layers.append(lay)
    return config(layers, width=rng.choice([40, 56, 100, 136, 192]), vocab=rng.randint(30, 400), alpha=rng.choice([1.0, 0.7, 2.2]),
                  scale=rng.uniform(0.3, 2.0), buckets=rng.randint(3, 5000), mul_prev=rng.randint(0, 10 ** 6), mul_cur=rng.randint(0, 10 ** 6),
                  eps=rng.choice([1e-6, 1e-5, 1e-3]))


@pytest.mark.parametrize("seed", list(range(8)))
def test_configurations_drawn_at_random(device, tmp_path, seed):
    """Whole prompts in one batch, then a prompt in portions with its last tokens one by one beside another request, in
    both precisions, for sizes nobody chose."""
    c = random_config(seed)
    weights = make_weights(c, seed=100 + seed)
    folder = write_folder(tmp_path, c, weights)
    g = torch.Generator().manual_seed(seed)
    tokens = {"a": torch.randint(0, c["vocab"], (83,), generator=g).tolist(), "b": torch.randint(0, c["vocab"], (21,), generator=g).tolist()}
    want = {k: plain.forward(c, weights, v).numpy() for k, v in tokens.items()}
    for dtype in ("float32", "bfloat16"):
        d = Driver(folder, dtype, pages=40, page_size=4, max_requests=2)
        whole = d.run([[("a", 83), ("b", 21)]], tokens)
        cut = d.run([[("a", 30)], [("a", 17), ("b", 2)], [("a", 2), ("b", 1)], [("a", 24), ("b", 9)]] + [[("a", 1), ("b", 1)]] * 10, tokens)
        for got in (whole, cut):
            check_rows(np.concatenate([row_error(got[k], want[k]) for k in tokens]), dtype, (seed, c["width"]))
        d.close()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_prompt_in_one_step(device, tmp_path, dtype):
    """1,700 tokens: 1,500 in one step (retention in several segments a sequence, prompt attention over many tiles),
    then a portion of 150 behind them and single tokens, beside a second, short request."""
    c = CONFIGS["odd"]
    weights = make_weights(c, seed=17)
    folder = write_folder(tmp_path, c, weights)
    g = torch.Generator().manual_seed(6)
    tokens = {"a": torch.randint(0, c["vocab"], (1700,), generator=g).tolist(), "b": torch.randint(0, c["vocab"], (40,), generator=g).tolist()}
    want = {k: plain.forward(c, weights, v).numpy() for k, v in tokens.items()}
    d = Driver(folder, dtype, pages=120, page_size=16, max_requests=2)
    got = d.run([[("a", 1500), ("b", 3)], [("a", 150), ("b", 1)]] + [[("a", 1), ("b", 1)]] * 36 + [[("a", 14)]], tokens)
    check_rows(np.concatenate([row_error(got[k], want[k]) for k in tokens]), dtype)
    d.close()


def test_long_decoding_from_graphs(device, tmp_path):
    """400 tokens decoded one by one from graphs after a short prompt, two requests side by side."""
    c = CONFIGS["odd"]
    weights = make_weights(c, seed=11)
    folder = write_folder(tmp_path, c, weights)
    g = torch.Generator().manual_seed(3)
    tokens = {"a": torch.randint(0, c["vocab"], (420,), generator=g).tolist(),
              "b": torch.randint(0, c["vocab"], (409,), generator=g).tolist()}
    want = {k: plain.forward(c, weights, v).numpy() for k, v in tokens.items()}
    d = Driver(folder, "float32", pages=70, page_size=16)
    got = d.run([[("a", 20), ("b", 9)]] + [[("a", 1), ("b", 1)] for _ in range(400)], tokens)
    for k in tokens:
        err = row_error(got[k], want[k])
        assert err.max() < BAR["float32"], (k, int(err.argmax()), float(err.max()))
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

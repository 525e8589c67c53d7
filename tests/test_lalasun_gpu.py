"""Lalasun on the GPU against the plain statement in ``oracle/lalasun.py``: every mechanism alone, then whole
models through the engine -- whole prompts, token-by-token decoding, portions down to two tokens, mixed batches,
pages and state slots that are reused, greedy generation through ``LLM.generate``, the replay entry point.

The models are small and random (``tests/lalasun_util.py``); where random numbers would hide a fault (one far key
among hundreds, a key on a page border, at a window's or a chunk's edge, a missing softmax sink) the inputs are
built so that it shows.
"""
import random
from types import SimpleNamespace

import pytest
import torch

import lalasun_util as lu
from oracle import lalasun as oracle

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F64 = torch.float64


def ragged(seqs, width=None):
    """seqs: [(ctx_len, new tokens, state slot, block table)] -> the step's ragged layout on the device."""
    q_start, token_seq = [0], []
    for i, (_, n, _, _) in enumerate(seqs):
        q_start.append(q_start[-1] + n)
        token_seq += [i] * n
    width = width or max(len(s[3]) for s in seqs) or 1
    tables = [list(s[3]) + [0] * (width - len(s[3])) for s in seqs]
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)          # noqa: E731
    return SimpleNamespace(
        q_start=i32(q_start), ctx_len=i32([s[0] for s in seqs]), token_seq=i32(token_seq),
        state_slot=i32([s[2] for s in seqs]), block_tables=i32(tables).reshape(len(seqs), width), num_seqs=len(seqs),
        max_query_len=max(s[1] for s in seqs), max_pages_used=width,
        max_page_id=max([max(s[3]) for s in seqs if s[3]] or [0]), max_state_slot=max(s[2] for s in seqs))


def ops():
    from splitwise_amd import _C
    return _C.mixer_ops


def tol_of(dtype):
    return dict(atol=2e-5, rtol=2e-5) if dtype == torch.float32 else dict(atol=2e-2, rtol=2e-2)


# ------------------------------------------------------------------ mechanisms alone
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width", [48, 200, 1030, 2500])
def test_gated_stream_step(dtype, width):
    """The gated add, the filing into the history with the depth mix, and the tanh norm, in every combination."""
    g = torch.Generator().manual_seed(width)
    rows, entries = 7, 4
    x = torch.randn(rows, width, generator=g) * 3
    y = torch.randn(rows, 2 * width + 5, generator=g).to(dtype)
    y, gate = y[:, 5:5 + width], y[:, 5 + width:]                        # views with a row stride
    hist = torch.randn(entries, rows, width, generator=g)
    dw = torch.randn(entries, generator=g)
    alpha, w, b = torch.tensor([0.37]), torch.randn(width, generator=g), torch.randn(width, generator=g) * 0.2
    for use_y, use_gate, use_hist, use_norm in [(True, True, False, True), (True, True, True, True), (True, False, False, False),
                                                (False, False, False, True), (True, True, True, False), (False, False, True, True)]:
        for n_hist in ([1, 2, entries] if use_hist else [0]):
            stream = x.clone().to(DEV)
            hd = hist.clone().to(DEV)
            out = torch.empty(rows, width, dtype=dtype, device=DEV) if use_norm else None
            ops().gated_stream_step(stream, y.to(DEV) if use_y else None, gate.to(DEV) if use_gate else None, 0.6,
                                    hd[:n_hist] if use_hist else None, dw[:n_hist].contiguous().to(DEV) if use_hist else None,
                                    (alpha.to(DEV), w.to(DEV), b.to(DEV)) if use_norm else None, out)
            want = x.double()
            if use_y:
                want = want + 0.6 * y.double() * (torch.sigmoid(gate.double()) if use_gate else 1.0)
            if use_hist:
                torch.testing.assert_close(hd[n_hist - 1].cpu().double(), want, atol=1e-5, rtol=1e-6)
                torch.testing.assert_close(hd[n_hist:].cpu(), hist[n_hist:])              # later entries untouched
                want = sum(dw[j].double() * hist[j].double() for j in range(n_hist - 1)) + dw[n_hist - 1].double() * want
            torch.testing.assert_close(stream.cpu().double(), want, atol=2e-5, rtol=1e-6)
            if use_norm:
                torch.testing.assert_close(out.cpu().double(), oracle.tanh_norm(want, alpha.double(), w.double(), b.double()),
                                           **tol_of(dtype))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("ff,coef", [(40, (0.9, 0.4, -0.3, 0.1)), (320, (1.0, 0.0, 0.0, 0.0)), (2100, (0.0, 0.0, 1.0, -0.5)),
                                     (33, (0.2, 1.5, 0.7, 0.0))])
def test_poly_norm(dtype, ff, coef):
    g = torch.Generator().manual_seed(ff)
    z = (torch.randn(5, ff + 3, generator=g) * 1.7).to(dtype)[:, 3:]
    z[4] *= 1e-4                                                         # a row small enough for eps to count
    c = torch.tensor(coef)
    out = torch.empty(5, ff, dtype=dtype, device=DEV)
    ops().poly_norm(out, z.to(DEV), c.to(DEV), 1e-5)
    torch.testing.assert_close(out.cpu().double(), oracle.poly_norm(z.double(), c.double(), 1e-5), **tol_of(dtype))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gate_mul_and_head_norm_with_a_silu_gate(dtype):
    g = torch.Generator().manual_seed(3)
    rows, H, size = 6, 3, 20
    y = torch.randn(H, rows, size, generator=g).to(dtype)                # as a batched product over heads leaves it
    gate = torch.randn(rows, H * size + 2, generator=g).to(dtype)[:, 2:]
    for silu in (False, True):
        out = torch.empty(rows, H * size, dtype=dtype, device=DEV)
        ops().gate_mul(out, y.to(DEV).transpose(0, 1), gate.to(DEV), silu)
        f = gate.double() * torch.sigmoid(gate.double()) if silu else torch.sigmoid(gate.double())
        torch.testing.assert_close(out.cpu().double(), y.double().transpose(0, 1).reshape(rows, -1) * f, **tol_of(dtype))
    o = torch.randn(rows, H * size, generator=g) * 2
    w = torch.randn(size, generator=g)
    out = torch.empty(rows, H * size, dtype=dtype, device=DEV)
    ops().head_norm_gate(out, o.to(DEV), gate.to(DEV), w.to(DEV), False, 1e-5, H, size, gate_silu=True)
    want = (oracle.rms_unit(o.double().view(rows, H, size), 1e-5) * w.double()).reshape(rows, -1)
    torch.testing.assert_close(out.cpu().double(), want * gate.double() * torch.sigmoid(gate.double()), **tol_of(dtype))


@pytest.mark.parametrize("H,G,d,dv,rot", [(4, 2, 16, 8, 8), (3, 3, 8, 8, 8), (6, 2, 20, 24, 4), (2, 1, 80, 64, 80), (2, 2, 10, 6, 0)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rotation_by_halves_and_cache_write(H, G, d, dv, rot, dtype):
    from splitwise_amd.model_executor.layers.basic import rotary_frequencies
    g = torch.Generator().manual_seed(H * 100 + d)
    rows, page = 9, 16
    positions = torch.tensor([0, 1, 2, 15, 16, 17, 300, 2047, 70000])
    proj = torch.randn(rows, H * d + G * d + G * dv + 7, generator=g).to(dtype)
    q, k, v = proj[:, :H * d], proj[:, H * d:H * d + G * d], proj[:, H * d + G * d:H * d + G * d + G * dv]
    freqs = oracle.rotary_frequencies({"base": 50.0, "dims": rot}) if rot else []
    inv = rotary_frequencies(rot, 50.0) if rot else None
    slots = torch.tensor([40, 3, 17, 64, 65, 0, 99, 31, 32])
    kc = torch.zeros(8, page, G * d, dtype=dtype, device=DEV)
    vc = torch.zeros(8, page, G * dv, dtype=dtype, device=DEV)
    q_out = torch.empty(rows, H * d, dtype=torch.float32, device=DEV)
    dev = proj.to(DEV)
    ops().rope_cache(q_out, dev[:, :H * d], dev[:, H * d:H * d + G * d], dev[:, H * d + G * d:H * d + G * d + G * dv],
                     positions.to(DEV), None if inv is None else inv.to(DEV), H, G, d, dv, kc, vc, slots.to(DEV), True)
    for t in range(rows):
        want_q = oracle.rotate_halves(q[t].double().view(H, d), int(positions[t]), freqs).reshape(-1)
        want_k = oracle.rotate_halves(k[t].double().view(G, d), int(positions[t]), freqs).reshape(-1)
        torch.testing.assert_close(q_out[t].cpu().double(), want_q, atol=2e-5, rtol=2e-5)
        torch.testing.assert_close(kc.view(-1, G * d)[slots[t]].cpu().double(), want_k, **tol_of(dtype))
        torch.testing.assert_close(vc.view(-1, G * dv)[slots[t]].cpu(), v[t])
    if rot and rot < d:
        # halves and neighbours are different rotations: the flag must matter
        q2 = torch.empty_like(q_out)
        ops().rope_cache(q2, dev[:, :H * d], None, None, positions.to(DEV), inv.to(DEV), H, G, d, dv, None, None, None, False)
        assert (q2 - q_out).abs().max() > 1e-2


@pytest.mark.parametrize("H,rank,rot", [(3, 20, 4), (1, 8, 2), (4, 64, 16), (2, 130, 6), (2, 12, 0)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_latent_rows_and_query_layout(H, rank, rot, dtype):
    from splitwise_amd.model_executor.layers.basic import rotary_frequencies
    g = torch.Generator().manual_seed(rank)
    rows, page = 7, 8
    positions = torch.tensor([0, 1, 7, 8, 9, 300, 50000])
    q_latent = torch.randn(H, rows, rank, generator=g).to(dtype)
    proj = torch.randn(rows, H * (5 + rot) + rank + rot + 3, generator=g).to(dtype)
    per_head = proj[:, :H * (5 + rot)].unflatten(1, (H, 5 + rot))
    down = proj[:, H * (5 + rot):H * (5 + rot) + rank + rot]
    down[6, :rank] *= 1e-3                                               # a latent small enough for eps to count
    w = torch.randn(rank, generator=g) * 0.3 + 1.0
    freqs = oracle.rotary_frequencies({"base": 30.0, "dims": rot}) if rot else []
    inv = rotary_frequencies(rot, 30.0).to(DEV) if rot else torch.zeros(0, device=DEV)
    slots = torch.tensor([9, 0, 17, 31, 16, 8, 2])
    cache = torch.zeros(4, page, rank + rot, dtype=dtype, device=DEV)
    q_out = torch.empty(rows, H * (rank + rot), dtype=torch.float32, device=DEV)
    pd = proj.to(DEV)
    ops().latent_rope_cache(q_out, q_latent.to(DEV).transpose(0, 1), pd[:, :H * (5 + rot)].unflatten(1, (H, 5 + rot))[:, :, 5:],
                            pd[:, H * (5 + rot):H * (5 + rot) + rank + rot], w.to(DEV), 1e-5, positions.to(DEV), inv, cache,
                            slots.to(DEV))
    got_q = q_out.cpu().double().view(rows, H, rank + rot)
    for t in range(rows):
        pos = int(positions[t])
        torch.testing.assert_close(got_q[t, :, :rank], q_latent[:, t].double(), atol=0, rtol=0)
        torch.testing.assert_close(got_q[t, :, rank:], oracle.rotate_neighbours(per_head[t, :, 5:].double(), pos, freqs),
                                   atol=2e-5, rtol=2e-5)
        row = cache.view(-1, rank + rot)[slots[t]].cpu().double()
        torch.testing.assert_close(row[:rank], oracle.rms_unit(down[t, :rank].double(), 1e-5) * w.double(), **tol_of(dtype))
        torch.testing.assert_close(row[rank:], oracle.rotate_neighbours(down[t:t + 1, rank:].double(), pos, freqs)[0],
                                   **tol_of(dtype))


def _attention_case(H, G, d, dv, n, spikes, seed, big=6.0):
    """Random q, k, v with, for every (query position, key position, head) in ``spikes``, that query and key made
    long along a direction of their own, so that the pair's score towers over the query's other scores."""
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(n, H, d, generator=g) * 0.5
    k = torch.randn(n, G, d, generator=g) * 0.5
    v = torch.randn(n, G, dv, generator=g)
    for num, (i, j, a) in enumerate(spikes):
        e = torch.zeros(d)
        e[num % d] = 1.0
        q[i, a] = big * e + 0.05 * q[i, a]
        k[j, a // (H // G)] = big * e + 0.05 * k[j, a // (H // G)]
    return q, k, v


def _paged(rows_k, rows_v, page, dtype, seed):
    """Key / value rows in pages handed out in a shuffled order; unused pages hold NaN."""
    n = rows_k.shape[0]
    pages = -(-n // page)
    order = list(range(pages + 3))
    random.Random(seed).shuffle(order)
    table = order[:pages]
    kc = torch.full((pages + 3, page, rows_k.shape[1]), float("nan"), dtype=dtype)
    vc = None if rows_v is None else torch.full((pages + 3, page, rows_v.shape[1]), float("nan"), dtype=dtype)
    for t in range(n):
        kc[table[t // page], t % page] = rows_k[t].to(dtype)
        if vc is not None:
            vc[table[t // page], t % page] = rows_v[t].to(dtype)
    return kc.to(DEV), None if vc is None else vc.to(DEV), table


def _steps_of(mode, n, table):
    """-> (the step's sequences, the positions they cover in order)."""
    if mode == "prompt":
        return [(0, n, 0, table)], list(range(n))
    if mode == "decode":
        rows = list(range(n - 45, n)) + [0, 1, 33]
        return [(t, 1, 0, table) for t in rows], rows
    if mode == "pairs":                                                  # steps of two tokens, and one of a single token
        firsts = list(range(n - 46, n, 2)) + [0, 32, 127]
        return [(t, 2, 0, table) for t in firsts] + [(n - 47, 1, 0, table)], \
            [t + i for t in firsts for i in range(2)] + [n - 47]
    cuts, at = [], 0
    for size in [3, 2, 27, 1, 31, 2, 64, 2, 33, 5, 32, 98]:
        cuts.append((at, size, 0, table))
        at += size
    assert at == n
    random.Random(3).shuffle(cuts)                                       # portions of "different sequences" in any order
    return cuts, [c[0] + i for c in cuts for i in range(c[1])]


@pytest.mark.parametrize("H,G,d,dv,page", [(4, 2, 16, 8, 16), (6, 6, 8, 8, 16), (3, 1, 24, 72, 8), (8, 2, 20, 40, 16),
                                           (2, 1, 128, 128, 64), (4, 4, 64, 16, 32)])
@pytest.mark.parametrize("mode", ["prompt", "decode", "pairs", "portions"])
@pytest.mark.parametrize("cache_dtype,chunk,sink", [(torch.float32, 37, True), (torch.bfloat16, 37, True), (torch.float32, 64, False),
                                                    (torch.float32, 0, True), (torch.float32, 1000, True)])
def test_chunked_attention_with_a_sink(H, G, d, dv, page, mode, cache_dtype, chunk, sink):
    n = 300
    last = n - 1
    # keys on both sides of a page border and of a 32-key tile, the query's own key; with chunks: a chunk's first
    # position seen from its last one, and the position before it, which belongs to the chunk before and must not be seen
    spikes = [(last - 1, last - 3, H - 1), (last - 5, last - 5, H - 1), (128, 128, 0), (40, 39, H - 1)]
    if chunk:
        c = chunk
        start = last // c * c
        spikes += [(last, start, 0), (last - 2, max(start - 1, 0), H - 1), (2 * c - 1, c, 0), (2 * c - 2, c - 1, H - 1),
                   (c, c - 1, 0), (c - 1, 0, H - 1)]
        spikes = [s for s in spikes if 0 <= s[1] <= s[0] < n]
    else:
        spikes += [(last, 2, 0), (last - 2, page, 0), (last - 3, 31, H - 1), (100, 0, 0)]
    q, k, v = _attention_case(H, G, d, dv, n, spikes, seed=H * 1000 + d)
    q[7] *= 0.01                                                         # a row whose scores are near 0: the sink weighs most
    kc, vc, table = _paged(k.reshape(n, -1), v.reshape(n, -1), page, cache_dtype, seed=d)
    kk = torch.stack([kc.cpu().double()[table[t // page], t % page].view(G, d) for t in range(n)])
    vv = torch.stack([vc.cpu().double()[table[t // page], t % page].view(G, dv) for t in range(n)])
    scale = 0.9
    want = oracle.masked_attention(q.double(), kk, vv, scale, chunk=chunk, sink=sink).reshape(n, H * dv)
    if sink:                                                             # the test would not notice a missing sink otherwise
        plain = oracle.masked_attention(q[:9].double(), kk, vv, scale, chunk=chunk).reshape(9, H * dv)
        assert (plain - want[:9]).abs().max() > 0.05
    seqs, rows = _steps_of(mode, n, table)
    batch = ragged(seqs)
    qd = q[rows].reshape(len(rows), H * d).contiguous().to(DEV)
    out = torch.empty(len(rows), H * dv, dtype=cache_dtype, device=DEV)
    ops().capped_attention(out, qd, kc, vc, None, batch, H, G, d, dv, scale, 0.0, 0, chunk, sink)
    tol = dict(atol=3e-5, rtol=3e-5) if cache_dtype == torch.float32 else dict(atol=2e-2, rtol=2e-2)
    torch.testing.assert_close(out.cpu().double(), want[rows], **tol)


@pytest.mark.parametrize("H,rank,rot,page", [(3, 20, 4, 16), (4, 64, 16, 16), (2, 130, 6, 8), (1, 8, 2, 32), (8, 40, 8, 16),
                                             (2, 288, 32, 16), (16, 24, 8, 16), (2, 450, 32, 16)])
@pytest.mark.parametrize("mode", ["prompt", "decode", "pairs", "portions"])
@pytest.mark.parametrize("cache_dtype,window", [(torch.float32, 37), (torch.bfloat16, 37), (torch.float32, 0), (torch.float32, 1)])
def test_attention_over_a_shared_latent(H, rank, rot, page, mode, cache_dtype, window):
    """All heads read ONE key row per token and take its first ``rank`` numbers as the value."""
    n = 300
    last = n - 1
    d = rank + rot
    spikes = [(last, 2, 0), (last - 1, page - 1, H - 1), (last - 2, page, 0), (last - 3, 31, H - 1), (last - 4, 32, 0),
              (last - 5, last - 5, H - 1), (100, 0, 0), (129, 127, H - 1), (128, 128, 0), (40, 39, H - 1)]
    if window:
        spikes += [(last - 6, last - 6 - window + 1, 0), (last - 7, last - 7 - window, H - 1), (200, 200 - window, 0),
                   (window - 1, 0, 0), (window, 0, H - 1)]
    q, k, _ = _attention_case(H, 1, d, 1, n, spikes, seed=H * 1000 + d)
    kc, _, table = _paged(k.reshape(n, d), None, page, cache_dtype, seed=d)
    kk = torch.stack([kc.cpu().double()[table[t // page], t % page].view(1, d) for t in range(n)])
    scale = 0.9
    want = oracle.masked_attention(q.double(), kk, kk[:, :, :rank], scale, window=window).reshape(n, H * rank)
    seqs, rows = _steps_of(mode, n, table)
    batch = ragged(seqs)
    qd = q[rows].reshape(len(rows), H * d).contiguous().to(DEV)
    out = torch.empty(len(rows), H * rank, dtype=cache_dtype, device=DEV)
    ops().capped_attention(out, qd, kc, None, None, batch, H, 1, d, rank, scale, 0.0, window)
    tol = dict(atol=3e-5, rtol=3e-5) if cache_dtype == torch.float32 else dict(atol=2e-2, rtol=2e-2)
    torch.testing.assert_close(out.cpu().double(), want[rows], **tol)


@pytest.mark.parametrize("cache_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("kind", ["latent", "grouped"])
def test_decode_steps_of_few_sequences_share_their_keys_among_workgroups(kind, cache_dtype):
    """Three sequences with long contexts and sixteen query heads per key row: the keys of each are shared out among
    several workgroups whose parts a second launch joins.  A far key towers, one part sees no key at all (a window),
    and the sink and the gate are applied once, by the join."""
    n, page, H = 1500, 16, 16
    rank, rot = (40, 8) if kind == "latent" else (0, 0)
    d, dv = (rank + rot, rank) if kind == "latent" else (24, 40)
    rows = [n - 1, 1201, 700]
    spikes = [(n - 1, 3, 0), (1201, 1201 - 99, H - 1), (700, 650, 5)]
    q, k, v = _attention_case(H, 1, d, dv, n, spikes, seed=77)
    if kind == "latent":
        kc, vc, table = _paged(k.reshape(n, d), None, page, cache_dtype, seed=5)
    else:
        kc, vc, table = _paged(k.reshape(n, d), v.reshape(n, dv), page, cache_dtype, seed=5)
    kk = torch.stack([kc.cpu().double()[table[t // page], t % page].view(1, d) for t in range(n)])
    vv = kk[:, :, :rank] if kind == "latent" else torch.stack([vc.cpu().double()[table[t // page], t % page].view(1, dv) for t in range(n)])
    gate = torch.randn(len(rows), H * dv + 3, generator=torch.Generator().manual_seed(2)).to(cache_dtype)[:, 3:]
    batch = ragged([(t, 1, 0, table) for t in rows])
    qd = q[rows].reshape(len(rows), H * d).contiguous().to(DEV)
    from splitwise_amd import _C_mixers
    for window, chunk, sink, use_gate in [(0, 0, False, False), (100, 0, False, True), (0, 0, True, True), (0, 1100, True, False)]:
        need = _C_mixers.load_library().swm_masked_attention_workspace_floats(len(rows), len(rows), 1, H, 1, dv, page, len(table),
                                                                              window, chunk)
        assert (need > 0) == (window == 0)                      # a short window leaves too few keys to share out
        want = torch.stack([oracle.masked_attention(q[t:t + 1].double(), kk, vv, 0.9, window=window, chunk=chunk, sink=sink,
                                                    first_position=t)[0] for t in rows]).reshape(len(rows), H * dv)
        if use_gate:
            want = want * torch.sigmoid(gate.double())
        out = torch.empty(len(rows), H * dv, dtype=cache_dtype, device=DEV)
        ops().capped_attention(out, qd, kc, None if kind == "latent" else vc, gate.to(DEV) if use_gate else None, batch, H, 1, d, dv,
                               0.9, 0.0, window, chunk, sink)
        tol = dict(atol=3e-5, rtol=3e-5) if cache_dtype == torch.float32 else dict(atol=2e-2, rtol=2e-2)
        torch.testing.assert_close(out.cpu().double(), want, **tol)


def _run_gla(proj, sizes, bias, tau, state, steps, H, d, dv):
    """steps: [[(sequence, first token, tokens, slot)]]; proj[s]: the sequence's projections [n, q | k | v | z]."""
    nk, nv = sizes
    outs = {s: torch.zeros(p.shape[0], nv, dtype=torch.float32) for s, p in proj.items()}
    for step in steps:
        x = torch.cat([proj[s][lo:lo + n] for s, lo, n, _ in step]).to(DEV)
        batch = ragged([(lo, n, slot, []) for _, lo, n, slot in step], width=1)
        o = torch.empty(x.shape[0], nv, dtype=torch.float32, device=DEV)
        z = x[:, 2 * nk + nv:2 * nk + nv + nk].contiguous()
        ops().gla(o, x[:, :nk], x[:, nk:2 * nk], x[:, 2 * nk:2 * nk + nv], z, bias, tau, d ** -0.5, state, batch, H, d, dv)
        at = 0
        for s, lo, n, _ in step:
            outs[s][lo:lo + n] = o[at:at + n].cpu()
            at += n
    return outs


@pytest.mark.parametrize("H,d,dv,tau,shift", [(3, 24, 16, 4.0, 1.0), (1, 8, 8, 12.0, 3.0), (2, 64, 48, 1.0, -2.0), (2, 100, 48, 0.25, -4.0),
                                              (4, 40, 130, 2.0, 0.0), (1, 256, 64, 8.0, 2.0), (2, 32, 32, 0.05, -3.0)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gated_linear_attention_recurrence(H, d, dv, tau, shift, dtype):
    """Two sequences interleaved over three state slots that held other sequences before: whole chunks, chunk
    borders (31, 32, 33 tokens), portions of one and two tokens, a first portion of one token, a long run from a
    carried state beside a single token of the other sequence, and 70 tokens decoded one by one; against the
    recurrence run token by token in double precision.  The decays go from nearly 1 (large tau, positive shift) to
    products over a chunk far below the smallest float (small tau, negative shift)."""
    g = torch.Generator().manual_seed(H * 100 + d)
    nk, nv = H * d, H * dv
    lens = {"a": 640, "b": 139}
    proj = {}
    for s, n in lens.items():
        p = torch.randn(n, 3 * nk + nv + 3, generator=g) * 1.2
        p[:, 2 * nk + nv:] *= 2.0                                        # decay projections spread over several units
        proj[s] = p.to(dtype)
    bias = (torch.randn(nk, generator=g) + shift).to(DEV)
    state = torch.full((3, H, d, dv), float("nan"), dtype=torch.float32, device=DEV)     # slots are never cleared
    steps = [[("a", 0, 1, 2)], [("a", 1, 31, 2), ("b", 0, 33, 0)], [("b", 33, 2, 0), ("a", 32, 32, 2)],
             [("a", 64, 33, 2)], [("a", 97, 2, 2), ("b", 35, 64, 0)], [("a", 99, 471, 2), ("b", 99, 1, 0)]]
    steps += [[("a", 570 + i, 1, 2)] + ([("b", 100 + i, 1, 0)] if i < 39 else []) for i in range(70)]
    outs = _run_gla(proj, (nk, nv), bias, tau, state, steps, H, d, dv)
    final = {}
    for s, n in lens.items():
        p = proj[s].double()
        decay = oracle.channel_decay(p[:, 2 * nk + nv:2 * nk + nv + nk] + bias.cpu().double(), tau).view(n, H, d)
        want, final[s] = oracle.decayed_state_scan(p[:, :nk].view(n, H, d) * d ** -0.5, p[:, nk:2 * nk].view(n, H, d),
                                                   p[:, 2 * nk:2 * nk + nv].view(n, H, dv), decay)
        scale = want.abs().max()
        assert (outs[s].double() - want.reshape(n, nv)).abs().max() < 2e-5 * scale, s
    assert (state[2].cpu().double() - final["a"]).abs().max() < 2e-5 * final["a"].abs().max()
    assert (state[0].cpu().double() - final["b"]).abs().max() < 2e-5 * final["b"].abs().max()
    # a new sequence in a used slot starts from nothing, and one long run equals the portions
    whole = _run_gla(proj, (nk, nv), bias, tau, state, [[("b", 0, lens["b"], 2), ("a", 0, lens["a"], 1)]], H, d, dv)
    for s in lens:
        assert (whole[s] - outs[s]).abs().max() < 2e-5 * outs[s].abs().max()
    assert (state[1].cpu().double() - final["a"]).abs().max() < 2e-5 * final["a"].abs().max()


# --------------------------------------------------------------- whole models through the engine
def _cfg_a():
    layers = [lu.gla(2, 12, 20, 4.0), lu.latent(3, 8, 4, 12, 20, window=9), lu.attention(4, 2, 16, 8, chunk=11, rot_dims=8),
              lu.latent(2, 16, 8, 8, 24, window=45, scale=0.2), lu.gla(3, 8, 8, 12.0), lu.attention(2, 2, 12, 12, chunk=32, rot_dims=12)]
    mlps = [lu.dense(40), lu.dense(56), None, lu.dense(24), lu.dense(40), lu.dense(33)]
    return lu.config(layers, mlps, vocab=97, width=48, mult=0.8)


def _cfg_b():
    layers = [lu.attention(6, 2, 10, 14, chunk=7, scale=0.4, rot_dims=4, base=1000.0), lu.gla(1, 36, 8, 1.0),
              lu.latent(1, 12, 2, 20, 9, window=3, scale=0.5), lu.latent(4, 4, 6, 4, 40, window=1000, scale=0.45)]
    mlps = [None, lu.dense(30), lu.dense(8), None]
    return lu.config(layers, mlps, vocab=53, width=20, eps=1e-6, mult=1.0)


_CASES = {"a": (_cfg_a, 11), "b": (_cfg_b, 12)}
FP32_TOL = 2e-4


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    out = {}
    for name, (make, seed) in _CASES.items():
        cfg = make()
        sd = lu.random_weights(cfg, seed)
        path = lu.write_model(str(tmp_path_factory.mktemp("lalasun_" + name)), cfg, sd)
        g = torch.Generator().manual_seed(seed)
        reqs = {f"r{i}": torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()
                for i, n in enumerate([70, 41, 18, 1, 33, 52, 150])}
        want = {rid: oracle.logits(cfg, sd, toks, dtype=F64) for rid, toks in reqs.items()}
        out[name] = SimpleNamespace(cfg=cfg, sd=sd, path=path, reqs=reqs, want=want)
    return out


@pytest.fixture(scope="module")
def engines(models):
    cache = {}

    def get(name, dtype, **kw):
        key = (name, dtype, tuple(sorted(kw.items())))
        if key not in cache:
            cache[key] = lu.make_engine(models[name].path, dtype, **kw)
        return cache[key]
    return get


@pytest.mark.parametrize("name", ["a", "b"])
def test_stream_after_every_layer(models, engines, name):
    m = models[name]
    engine = engines(name, "float32")
    model = engine.model_executor.driver_worker.model_runner.model
    toks = m.reqs["r4"]
    _, want = oracle.logits(m.cfg, m.sd, toks, dtype=F64, keep_streams=True)
    model.keep_residuals = []
    try:
        lu.Replayer(engine, {"r4": toks}).run_alone("r4", [len(toks)])
        got = [r.cpu().double() for r in model.keep_residuals]
    finally:
        model.keep_residuals = None
    assert len(got) == len(want)
    for i, (a, b) in enumerate(zip(got, want)):
        assert (a - b).abs().max() < 1e-4 * b.abs().max(), f"layer {i} ({m.cfg['layers'][i]['type']})"


@pytest.mark.parametrize("name", ["a", "b"])
def test_whole_prompts_match_the_plain_statement(models, engines, name):
    m = models[name]
    for rid, toks in m.reqs.items():
        got = lu.Replayer(engines(name, "float32"), {rid: toks}).run_alone(rid, [len(toks)])
        assert lu.row_error(got, m.want[rid]) < FP32_TOL, rid


@pytest.mark.parametrize("name", ["a", "b"])
def test_decoding_token_by_token(models, engines, name):
    """Most of a prompt at once and then 45 (and 100) tokens one by one -- windows and chunks pass over decoded
    tokens --, and a sequence fed one token at a time from its very first."""
    m = models[name]
    for rid, first in (("r0", 25), ("r6", 50)):
        toks = m.reqs[rid]
        got = lu.Replayer(engines(name, "float32"), {rid: toks}).run_alone(rid, [first] + [1] * (len(toks) - first))
        assert lu.row_error(got, m.want[rid]) < FP32_TOL
    toks = m.reqs["r2"]
    got = lu.Replayer(engines(name, "float32"), {"r2": toks}).run_alone("r2", [1] * len(toks))
    assert lu.row_error(got, m.want["r2"]) < FP32_TOL


@pytest.mark.parametrize("name", ["a", "b"])
@pytest.mark.parametrize("portions", [[2] * 35, [3, 2, 16, 1, 2, 7, 17, 2, 2, 18], [15, 1, 16, 17, 2, 19], [33, 31, 2, 4]])
def test_portions_of_prompts(models, engines, name, portions):
    m = models[name]
    toks = m.reqs["r0"]
    assert sum(portions) == len(toks)
    got = lu.Replayer(engines(name, "float32"), {"r0": toks}).run_alone("r0", portions)
    assert lu.row_error(got, m.want["r0"]) < FP32_TOL


@pytest.mark.parametrize("name,dtype,tol", [("a", "float32", FP32_TOL), ("b", "float32", FP32_TOL), ("a", "bfloat16", 0.08)])
def test_mixed_batches_reuse_pages_and_slots(models, engines, name, dtype, tol):
    """Six unequal requests over three state slots and a pool of 9 pages: portions beside single tokens, requests
    that sit out steps, pages and slots handed on as requests end.  Every request must come out as it does alone."""
    m = models[name]
    reqs = {r: t for r, t in m.reqs.items() if r != "r6"}
    engine = engines(name, dtype, max_tokens=144, max_requests=3)
    rp = lu.Replayer(engine, reqs)
    free_before = engine.scheduler.block_manager.get_num_free_gpu_blocks()
    steps = [{"r0": 3, "r2": 16}, {"r0": 16, "r2": 1, "r3": 1}, {"r0": 2, "r1": 29, "r2": 1}, {"r0": 17, "r1": 2},
             {"r0": 30, "r1": 1}, {"r1": 9, "r0": 1}, {"r0": 1, "r4": 20}]
    for step in steps:
        rp.step(step)
    rnd = random.Random(7)
    pending = ["r5"]
    while any(rp.at[r] < len(reqs[r]) for r in reqs):
        live = [r for r in rp.live if rp.at[r] < len(reqs[r])]
        while pending and len(live) < 3:
            nxt = pending[0]
            need = -(-len(reqs[nxt]) // 16)
            held = sum(-(-len(reqs[r]) // 16) for r in live)
            if held + need > 9:
                break
            live.append(pending.pop(0))
        step = {}
        for r in live:
            left = len(reqs[r]) - rp.at[r]
            step[r] = min(left, rnd.choice([1, 1, 2, 3, 16, 21]))
        if rnd.random() < 0.3 and len(step) > 1:
            step.pop(rnd.choice(sorted(step)))                  # somebody sits this step out
        rp.step(step)
    for rid in reqs:
        assert lu.row_error(rp.result(rid), m.want[rid]) < tol, rid
    assert engine.scheduler.block_manager.get_num_free_gpu_blocks() == free_before
    assert engine.scheduler.state_slots.num_free() == 3


def test_bfloat16_is_close_and_does_not_depend_on_the_cut(models, engines):
    m = models["a"]
    toks = m.reqs["r0"]
    whole = lu.Replayer(engines("a", "bfloat16"), {"r0": toks}).run_alone("r0", [len(toks)])
    cut = lu.Replayer(engines("a", "bfloat16"), {"r0": toks}).run_alone("r0", [2, 3, 16, 1, 1, 30, 17])
    assert lu.row_error(whole, m.want["r0"]) < 0.08
    assert lu.row_error(cut, m.want["r0"]) < 0.08
    assert lu.row_error(cut, whole) < 0.05


@pytest.mark.parametrize("name", ["a", "b"])
def test_greedy_generation_through_the_entry_point(models, name):
    """``LLM.generate`` with the scheduler's own policy: a token budget of 16 cuts the prompts into portions that
    run beside other requests' decoded tokens.  Every generated token must be (within rounding) the arg-max of
    the plain statement's logits for the text before it."""
    from splitwise_amd import LLM, SamplingParams
    m = models[name]
    llm = LLM(model=m.path, dtype="float32", block_size=16, max_model_len=128, max_num_seqs=3,
              max_num_batched_tokens=16, num_gpu_blocks_override=20, swap_space=0, enforce_eager=True)
    prompts = [m.reqs["r1"], m.reqs["r2"], m.reqs["r3"], m.reqs["r4"][:20]]
    outs = llm.generate(prompt_token_ids=prompts, sampling_params=SamplingParams(temperature=0.0, max_tokens=12,
                                                                                 ignore_eos=True))
    assert len(outs) == len(prompts)
    for prompt, out in zip(prompts, outs):
        new = out.outputs[0].token_ids
        assert len(new) == 12
        full = oracle.logits(m.cfg, m.sd, list(prompt) + list(new), dtype=F64)
        for k, tok in enumerate(new):
            row = full[len(prompt) + k - 1]
            assert row[tok] >= row.max() - 1e-3 * (row.max() - row.min()), (k, tok, int(row.argmax()))
    sched = llm.llm_engine.scheduler
    assert sched.state_slots.num_free() == 3 and not sched.running and not sched.waiting


def test_trace_run_replays_a_schedule(models, tmp_path):
    """``bin/trace_run`` as a user starts it: steps on standard input, ``done <step>`` after each, logits files in
    the order of the entries; requests that sit out a step, end, and hand their pages and slot on."""
    import json
    import os
    import subprocess
    import numpy as np
    m = models["b"]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    a, b, c = m.reqs["r1"], m.reqs["r2"], m.reqs["r4"]
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:7], "want": [0, 6]}, {"id": "b", "tokens": b[:2], "want": []}], "end": []},
        {"step": 1, "entries": [{"id": "b", "tokens": b[2:], "want": [15]}, {"id": "a", "tokens": a[7:8], "want": [0]}], "end": ["b"]},
        {"step": 2, "entries": [{"id": "a", "tokens": a[8:], "want": [len(a) - 9]}, {"id": "c", "tokens": c, "want": [0, len(c) - 1]}],
         "end": ["a", "c"]},
        {"step": 3, "entries": [{"id": "b", "tokens": b, "want": [len(b) - 1]}], "end": ["b"]},        # the name comes back
    ]
    out = tmp_path / "out"
    proc = subprocess.run([os.path.join(root, "bin", "trace_run"), "--model", m.path, "--dtype", "float32", "--out", str(out),
                           "--max-tokens", "128", "--max-requests", "2"],
                          input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [l for l in proc.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(4)]
    vocab = m.cfg["vocab"]
    want = {0: [m.want["r1"][0], m.want["r1"][6]], 1: [m.want["r2"][17], m.want["r1"][7]],
            2: [m.want["r1"][len(a) - 1], m.want["r4"][0], m.want["r4"][len(c) - 1]], 3: [m.want["r2"][len(b) - 1]]}
    for step, rows in want.items():
        got = torch.from_numpy(np.fromfile(out / f"{step}.f32", dtype="<f4").reshape(-1, vocab))
        assert got.shape[0] == len(rows)
        assert lu.row_error(got, torch.stack(rows)) < FP32_TOL, step

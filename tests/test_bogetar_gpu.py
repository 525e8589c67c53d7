"""Bogetar on the GPU against the plain statement in ``oracle/bogetar.py``: every mechanism alone, then whole
models through the engine -- whole prompts, token-by-token decoding, portions down to two tokens, mixed batches,
pages and state slots that are reused, greedy generation through ``LLM.generate``, the replay entry point.

The models are small and random (``tests/bogetar_util.py``); where random numbers would hide a fault (one far key
among hundreds, a key on a page border or at the window's edge, a group of experts that must not be chosen) the
inputs are built so that it shows.
"""
import random
from types import SimpleNamespace

import pytest
import torch

import bogetar_util as bu
from oracle import bogetar as oracle

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
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("y_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width,groups", [(48, 4), (48, 1), (200, 5), (1030, 2), (2560, 8), (66, 66)])
def test_group_norm_add(width, groups, y_dtype, out_dtype):
    """The norm of a sublayer's output into the stream, with layer scale, one or two addends, and the next norm."""
    g = torch.Generator().manual_seed(width + groups)
    rows, eps = 7, 1e-5
    x = torch.randn(rows, width, generator=g) * 3
    ys = torch.randn(rows, 2 * width + 5, generator=g).to(y_dtype)
    y1, y2 = ys[:, 5:5 + width], ys[:, 5 + width:]                       # views with a row stride
    y1[3] *= 1e-3                                                        # a row small enough for eps to count
    wb, ls, w = (torch.randn(width, generator=g) * 0.3 + 1.0 for _ in range(3))
    for use_y, use_y2, use_ls, use_out in [(True, False, True, True), (True, True, True, True), (True, True, False, False),
                                           (False, False, False, True), (True, False, False, True)]:
        stream = x.clone().to(DEV)
        out = torch.empty(rows, width, dtype=out_dtype, device=DEV) if use_out else None
        ops().group_norm_add(stream, groups, eps, y1.to(DEV) if use_y else None, wb.to(DEV) if use_y else None,
                             ls.to(DEV) if use_ls else None, y2.to(DEV) if use_y2 else None, 0.7, -1.3,
                             w.to(DEV) if use_out else None, out)
        want = x.double()
        if use_y:
            u = 0.7 * y1.double() + (-1.3 * y2.double() if use_y2 else 0.0)
            want = want + oracle.group_norm(u, wb.double(), groups, eps) * (ls.double() if use_ls else 1.0)
        torch.testing.assert_close(stream.cpu().double(), want, atol=3e-5, rtol=1e-5)
        if use_out:
            torch.testing.assert_close(out.cpu().double(), oracle.group_norm(want, w.double(), groups, eps),
                                       **tol_of(out_dtype))


def test_groups_matter():
    """The same row normed in one group and in four differs: a test with one group would not see the grouping."""
    x = torch.randn(3, 64, generator=torch.Generator().manual_seed(1)) * torch.linspace(0.1, 5.0, 64)
    w = torch.ones(64, dtype=F64)
    assert (oracle.group_norm(x.double(), w, 1, 1e-5) - oracle.group_norm(x.double(), w, 4, 1e-5)).abs().max() > 0.3


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("x_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("channels,taps", [(48, 3), (300, 2), (20, 5), (64, 1), (1000, 4)])
def test_convolution_added_to_its_input(channels, taps, x_dtype, out_dtype):
    """Two sequences interleaved over three slots that held other sequences before (and hold NaN where nothing was
    written): portions shorter than the taps, of one and two tokens, a first portion of one token, a slot used again."""
    g = torch.Generator().manual_seed(channels + taps)
    lens = {"a": 41, "b": 23}
    xs = {s: (torch.randn(n, channels + 3, generator=g) * 2).to(x_dtype)[:, 3:] for s, n in lens.items()}
    w = torch.randn(channels, taps, generator=g) * 0.5
    state = torch.full((3, taps - 1, channels), float("nan"), dtype=torch.float32, device=DEV)
    steps = [[("a", 0, 1, 2)], [("a", 1, 2, 2), ("b", 0, 3, 0)], [("b", 3, 1, 0), ("a", 3, 1, 2)], [("a", 4, 17, 2)],
             [("b", 4, 2, 0), ("a", 21, 2, 2)], [("a", 23, 18, 2), ("b", 6, 17, 0)]]
    got = {s: torch.zeros(n, channels, dtype=F64) for s, n in lens.items()}

    def run(steps, got):
        for step in steps:
            x = torch.cat([xs[s][lo:lo + n] for s, lo, n, _ in step]).to(DEV)
            out = torch.empty(x.shape, dtype=out_dtype, device=DEV)
            ops().causal_conv(out, x, w.to(DEV), state, ragged([(lo, n, slot, []) for _, lo, n, slot in step], width=1))
            at = 0
            for s, lo, n, _ in step:
                got[s][lo:lo + n] = out[at:at + n].cpu().double()
                at += n
    run(steps, got)
    for s in lens:
        x = xs[s].double()
        torch.testing.assert_close(got[s], x + oracle.causal_conv(x, w.double()), **tol_of(out_dtype))
    # a new sequence in used slots starts from nothing
    again = {s: torch.zeros(n, channels, dtype=F64) for s, n in lens.items()}
    run([[("b", 0, lens["b"], 2), ("a", 0, lens["a"], 0)]], again)
    for s in lens:
        torch.testing.assert_close(again[s], got[s], **tol_of(out_dtype))


@pytest.mark.parametrize("H,G,d,dv,rot", [(4, 2, 16, 8, 8), (3, 3, 8, 8, 8), (6, 2, 20, 24, 4), (2, 1, 80, 64, 80), (2, 2, 10, 6, 0)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_head_norm_rotation_and_cache_write(H, G, d, dv, rot, dtype):
    """Every query and key head normed over its coordinates with one weight for all heads, THEN rotated by halves."""
    from splitwise_amd.model_executor.layers.basic import rotary_frequencies
    g = torch.Generator().manual_seed(H * 100 + d)
    rows, page, eps = 9, 16, 1e-5
    proj = (torch.randn(rows, H * d + G * d + G * dv + 2, generator=g) * 1.5).to(dtype)
    q, k, v = proj[:, 2:2 + H * d], proj[:, 2 + H * d:2 + (H + G) * d], proj[:, 2 + (H + G) * d:]
    positions = torch.tensor([0, 1, 2, 70000, 5, 31, 1000, 7, 8])
    slots = torch.tensor([3, 17, 40, 41, -1, 2, 63, 16, 15])
    qw, kw = torch.randn(d, generator=g) * 0.3 + 1.0, torch.randn(d, generator=g) * 0.3 + 1.0
    freqs = rotary_frequencies(rot, 500.0) if rot else None
    kc = torch.zeros(4, page, G * d, dtype=dtype, device=DEV)
    vc = torch.zeros(4, page, G * dv, dtype=dtype, device=DEV)
    q32 = torch.empty(rows, H * d, dtype=torch.float32, device=DEV)
    pd = proj.to(DEV)
    ops().rope_cache(q32, pd[:, 2:2 + H * d], pd[:, 2 + H * d:2 + (H + G) * d], pd[:, 2 + (H + G) * d:], positions.to(DEV),
                     None if freqs is None else freqs.to(DEV), H, G, d, dv, kc, vc, slots.to(DEV), True, qw.to(DEV),
                     kw.to(DEV), eps)
    fl = oracle.rotary_frequencies({"base": 500.0, "dims": rot}) if rot else []

    def normed(u, w):
        return u / torch.sqrt(u.pow(2).mean(-1, keepdim=True) + eps) * w
    for t in range(rows):
        want_q = oracle.rotate_halves(normed(q[t].double().view(H, d), qw.double()), int(positions[t]), fl)
        torch.testing.assert_close(q32[t].cpu().double().view(H, d), want_q, atol=3e-5, rtol=3e-5)
        if slots[t] < 0:
            continue
        want_k = oracle.rotate_halves(normed(k[t].double().view(G, d), kw.double()), int(positions[t]), fl)
        torch.testing.assert_close(kc.view(-1, G, d)[slots[t]].cpu().double(), want_k, **tol_of(dtype))
        torch.testing.assert_close(vc.view(-1, G * dv)[slots[t]].cpu().double(), v[t].double(), atol=0, rtol=0)
    assert kc.view(-1, G * d)[4].abs().max() == 0                        # a row without a slot is not cached


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
    vc = torch.full((pages + 3, page, rows_v.shape[1]), float("nan"), dtype=dtype)
    for t in range(n):
        kc[table[t // page], t % page] = rows_k[t].to(dtype)
        vc[table[t // page], t % page] = rows_v[t].to(dtype)
    return kc.to(DEV), vc.to(DEV), table


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
                                           (2, 1, 128, 128, 64), (4, 4, 64, 16, 32), (16, 2, 12, 36, 16)])
@pytest.mark.parametrize("mode", ["prompt", "decode", "pairs", "portions"])
@pytest.mark.parametrize("cache_dtype,window,gated", [(torch.float32, 37, True), (torch.bfloat16, 37, False), (torch.float32, 0, False),
                                                      (torch.float32, 1, False), (torch.float32, 1000, True)])
def test_attention_with_sigmoid_weights(H, G, d, dv, page, mode, cache_dtype, window, gated):
    """No softmax: a towering key weighs 1 whatever else the query sees, so a key that is wrongly seen (one past the
    window) or wrongly missed (the window's last, a far one, one on a page border) changes the output by a whole value
    row.  The biases are negative, so the other keys weigh little; one head's bias is large to show that it is added."""
    n = 300
    last = n - 1
    spikes = [(last - 1, last - 3, H - 1), (last - 5, last - 5, H - 1), (128, 128, 0), (40, 39, H - 1), (129, 127, 0),
              (last - 2, page, 0), (last - 3, 31, H - 1), (100, 0, 0), (last, 2, 0), (last - 4, page - 1, H - 1)]
    if window:
        spikes += [(last - 6, last - 6 - window + 1, 0), (last - 7, last - 7 - window, H - 1), (200, 200 - window, 0),
                   (window - 1, 0, 0), (window, 0, H - 1), (250, 250 - window + 1, H - 1)]
        spikes = [s for s in spikes if 0 <= s[1] <= s[0] < n]
    q, k, v = _attention_case(H, G, d, dv, n, spikes, seed=H * 1000 + d)
    bias = torch.linspace(-4.0, -2.0, H)
    bias[H // 2] = 1.5
    kc, vc, table = _paged(k.reshape(n, -1), v.reshape(n, -1), page, cache_dtype, seed=d)
    kk = torch.stack([kc.cpu().double()[table[t // page], t % page].view(G, d) for t in range(n)])
    vv = torch.stack([vc.cpu().double()[table[t // page], t % page].view(G, dv) for t in range(n)])
    scale = 0.9
    want = oracle.sigmoid_window_attention(q.double(), kk, vv, bias.double(), scale, window or n + 1).reshape(n, H * dv)
    if 1 < window < n:                                                   # the test would not notice a window one off otherwise
        off = oracle.sigmoid_window_attention(q.double(), kk, vv, bias.double(), scale, window + 1).reshape(n, H * dv)
        assert (off - want).abs().max() > 0.5
    seqs, rows = _steps_of(mode, n, table)
    batch = ragged(seqs)
    qd = q[rows].reshape(len(rows), H * d).contiguous().to(DEV)
    gate = torch.randn(n, H * dv + 3, generator=torch.Generator().manual_seed(2)).to(cache_dtype)[:, 3:]
    if gated:
        want = want * torch.sigmoid(gate.double())
    out = torch.empty(len(rows), H * dv, dtype=cache_dtype, device=DEV)
    ops().capped_attention(out, qd, kc, vc, gate[rows].to(DEV) if gated else None, batch, H, G, d, dv, scale, 0.0, window,
                           score_bias=bias.to(DEV))
    tol = dict(atol=5e-5, rtol=5e-5) if cache_dtype == torch.float32 else dict(atol=3e-2, rtol=2e-2)
    torch.testing.assert_close(out.cpu().double(), want[rows], **tol)


@pytest.mark.parametrize("cache_dtype", [torch.float32, torch.bfloat16])
def test_sigmoid_weights_when_keys_are_shared_among_workgroups(cache_dtype):
    """Three sequences with long contexts and sixteen query heads per key head: the keys of each are shared out among
    several workgroups whose parts a second launch joins by plain addition; a far key towers; with a window one part
    sees no key at all."""
    n, page, H, d, dv = 1500, 16, 16, 24, 40
    rows = [n - 1, 1201, 700]
    spikes = [(n - 1, 3, 0), (1201, 1201 - 99, H - 1), (700, 650, 5)]
    q, k, v = _attention_case(H, 1, d, dv, n, spikes, seed=77)
    kc, vc, table = _paged(k.reshape(n, d), v.reshape(n, dv), page, cache_dtype, seed=5)
    kk = torch.stack([kc.cpu().double()[table[t // page], t % page].view(1, d) for t in range(n)])
    vv = torch.stack([vc.cpu().double()[table[t // page], t % page].view(1, dv) for t in range(n)])
    bias = torch.linspace(-6.0, -4.0, H)
    gate = torch.randn(len(rows), H * dv + 3, generator=torch.Generator().manual_seed(2)).to(cache_dtype)[:, 3:]
    batch = ragged([(t, 1, 0, table) for t in rows])
    qd = q[rows].reshape(len(rows), H * d).contiguous().to(DEV)
    from splitwise_amd import _C_mixers
    for window, use_gate in [(0, False), (1300, True), (100, True)]:
        need = _C_mixers.load_library().swm_masked_attention_workspace_floats(len(rows), len(rows), 1, H, 1, dv, page, len(table),
                                                                              window, 0)
        assert (need > 0) == (window != 100)                    # a short window leaves too few keys to share out
        want = torch.stack([oracle.sigmoid_window_attention(q[t:t + 1].double(), kk, vv, bias.double(), 0.9, window or n + 1,
                                                            first_position=t)[0] for t in rows]).reshape(len(rows), H * dv)
        if use_gate:
            want = want * torch.sigmoid(gate.double())
        out = torch.empty(len(rows), H * dv, dtype=cache_dtype, device=DEV)
        ops().capped_attention(out, qd, kc, vc, gate.to(DEV) if use_gate else None, batch, H, 1, d, dv, 0.9, 0.0, window,
                               score_bias=bias.to(DEV))
        tol = dict(atol=5e-5, rtol=5e-5) if cache_dtype == torch.float32 else dict(atol=3e-2, rtol=2e-2)
        torch.testing.assert_close(out.cpu().double(), want, **tol)


@pytest.mark.parametrize("H,G,d,dv,taps", [(3, 3, 12, 8, 4), (4, 2, 8, 20, 2), (1, 1, 64, 64, 4), (6, 1, 33, 10, 3), (2, 2, 130, 48, 5),
                                           (2, 1, 256, 16, 4)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("chunked", [None, True])
def test_delta_rule_with_one_decay_per_head(H, G, d, dv, taps, dtype, chunked):
    """The short convolution with silu, unit queries and keys, beta, the per-head decay and the rule itself: two
    sequences interleaved over three slots that hold NaN, portions of one and two tokens, 40 tokens decoded one by
    one; then both as whole prompts in other slots.  ``chunked`` None: steps that bring 32 tokens or more of a sequence
    go through the chunks of 32 on the matrix cores, the others token by token; True: every step goes through the
    chunks (a decoded token is a chunk of one, runs end inside chunks, the state passes from route to route)."""
    g = torch.Generator().manual_seed(H * 100 + d)
    c = 2 * G * d + H * dv
    lens = {"a": 150, "b": 61}
    proj = {s: (torch.randn(n, c + 2 * H + 1, generator=g) * 1.3).to(dtype)[:, 1:] for s, n in lens.items()}
    conv_w = torch.randn(c, taps, generator=g) * 0.6
    a_log, dt_bias = torch.randn(H, generator=g) * 0.7, torch.randn(H, generator=g)
    conv_state = torch.full((3, taps - 1, c), float("nan"), dtype=torch.float32, device=DEV)
    rule_state = torch.full((3, H, d, dv), float("nan"), dtype=torch.float32, device=DEV)

    def run(steps):
        outs = {s: torch.zeros(n, H * dv, dtype=F64) for s, n in lens.items()}
        for step in steps:
            x = torch.cat([proj[s][lo:lo + n] for s, lo, n, _ in step]).to(DEV)
            batch = ragged([(lo, n, slot, []) for _, lo, n, slot in step], width=1)
            qkv = torch.empty(x.shape[0], c, dtype=torch.float32, device=DEV)
            ops().causal_conv(qkv, x[:, :c], conv_w.to(DEV), conv_state, batch, silu=True, residual=False)
            o = torch.empty(x.shape[0], H * dv, dtype=torch.float32, device=DEV)
            ops().gated_delta(o, qkv, x[:, c:c + H], x[:, c + H:], dt_bias.to(DEV), a_log.to(DEV), rule_state, batch, H, G, d, dv,
                              chunked=chunked)
            at = 0
            for s, lo, n, _ in step:
                outs[s][lo:lo + n] = o[at:at + n].cpu().double()
                at += n
        return outs
    steps = [[("a", 0, 1, 2)], [("a", 1, 2, 2), ("b", 0, 3, 0)], [("b", 3, 2, 0), ("a", 3, 30, 2)], [("a", 33, 77, 2), ("b", 5, 1, 0)],
             [("b", 6, 15, 0)]]
    steps += [[("a", 110 + i, 1, 2), ("b", 21 + i, 1, 0)] for i in range(40)]
    outs = run(steps)
    final = {}
    for s, n in lens.items():
        p = proj[s].double()
        z = oracle.silu(oracle.causal_conv(p[:, :c], conv_w.double()))
        q = oracle.unit(z[:, :G * d].view(n, G, d)).repeat_interleave(H // G, 1) * d ** -0.5
        k = oracle.unit(z[:, G * d:2 * G * d].view(n, G, d)).repeat_interleave(H // G, 1)
        beta = torch.sigmoid(p[:, c:c + H])
        decay = torch.exp(-torch.exp(a_log.double()) * oracle.softplus(p[:, c + H:] + dt_bias.double()))
        want, final[s] = oracle.gated_delta_scan(q, k, z[:, 2 * G * d:].view(n, H, dv), beta, decay)
        assert (outs[s] - want.reshape(n, H * dv)).abs().max() < 3e-5 * max(want.abs().max(), 1.0), s
    assert (rule_state[2].cpu().double() - final["a"]).abs().max() < 3e-5 * max(final["a"].abs().max(), 1.0)
    whole = run([[("b", 0, lens["b"], 1), ("a", 0, lens["a"], 0)]])
    for s in lens:
        assert (whole[s] - outs[s]).abs().max() < 3e-5 * max(outs[s].abs().max(), 1.0)


@pytest.mark.parametrize("experts,top,groups,keep", [(6, 2, 3, 2), (8, 4, 4, 3), (8, 3, 1, 1), (12, 12, 4, 4), (5, 1, 5, 1), (64, 6, 8, 2)])
def test_softmax_router_with_groups(experts, top, groups, keep):
    """Logits built so that the limit to the best groups changes the choice: rows in which the second-best expert
    over all sits in a group that is dropped (the test asserts that such rows exist)."""
    g = torch.Generator().manual_seed(experts)
    rows = 200
    z = torch.randn(rows, experts, generator=g) * 2.0
    chosen, weights = ops().group_router(z.to(DEV), None, top, groups, keep, 1.0, True, True, False)
    changed = 0
    for t in range(rows):
        want_ids, want_w = oracle.route(z[t].double(), top, groups, keep)
        got = sorted(zip(chosen[t].tolist(), weights[t].tolist()))
        want = sorted(zip(want_ids.tolist(), want_w.tolist()))
        assert [e for e, _ in got] == [e for e, _ in want], t
        torch.testing.assert_close(torch.tensor([w for _, w in got]), torch.tensor([w for _, w in want]), atol=1e-6, rtol=1e-5)
        changed += sorted(torch.topk(z[t], top).indices.tolist()) != [e for e, _ in want]
    if keep < groups and keep < top < experts:          # with top <= keep the best experts sit in the best groups anyway
        assert changed > 0
    total = weights.sum(-1)
    assert bool((total <= 1.0 + 1e-5).all()) and (top == experts or bool((total < 0.999).any()))     # not renormalised


@pytest.mark.parametrize("dtype,width,ff", [(torch.float32, 48, 20), (torch.bfloat16, 48, 20), (torch.bfloat16, 64, 96), (torch.float32, 30, 7),
                                            (torch.bfloat16, 36, 10)])
def test_routed_experts_with_a_gated_hidden_layer(dtype, width, ff):
    from splitwise_amd.model_executor.layers.moe import GroupRoutedExperts
    g = torch.Generator().manual_seed(width + ff)
    experts, top, rows, limit = 6, 2, 90, 0.8
    mlp = {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top,
                                                                            "groups": {"count": 3, "keep": 2}}}
    w = {"router": torch.randn(experts, width, generator=g) * 3.0 / width ** 0.5}
    for e in range(experts):
        w[f"e{e}.gate"] = (torch.randn(ff, width, generator=g) * 2.0 / width ** 0.5).to(dtype)
        w[f"e{e}.up"] = (torch.randn(ff, width, generator=g) * 2.0 / width ** 0.5).to(dtype)
        w[f"e{e}.down"] = (torch.randn(width, ff, generator=g) / ff ** 0.5).to(dtype)
    layer = GroupRoutedExperts(width, experts, top, ff, None, 3, 2, 1.0, dtype, None, score="softmax", group_score="max",
                               normalize=False, activation="clamped_glu", limit=limit).to(DEV)
    layer.load_named({k: v.to(DEV) for k, v in w.items()})
    h = torch.randn(rows, width, generator=g).to(dtype)
    _, out = layer(h.to(DEV))
    hd = h.double()
    bites = (torch.stack([w[f"e{e}.gate"].double() @ hd.t() for e in range(experts)]) > limit).float().mean()
    assert 0.02 < bites < 0.9                                            # the limit bites, and not everywhere
    want = oracle.experts_ff(hd, {k: v.double() for k, v in w.items()}, mlp)
    tol = dict(atol=3e-5, rtol=3e-5) if dtype == torch.float32 else dict(atol=3e-2, rtol=3e-2)
    torch.testing.assert_close(out.cpu().double(), want, **tol)


# --------------------------------------------------------------- whole models through the engine
def _cfg_a():
    layers = [bu.parallel(4, 2, 16, 24, window=9, rot_dims=8), bu.delta(3, 3, 12, 8, conv=4),
              bu.parallel(6, 6, 8, 8, window=45, rot_dims=8, scale=0.4, r_heads=1, r_dim=20, r_vdim=16, tau=12.0, left_scale=1.0,
                          right_scale=0.4),
              bu.delta(4, 2, 10, 14, conv=2), bu.parallel(3, 1, 20, 12, window=17, rot_dims=4, base=1000.0, r_heads=2, r_dim=8, r_vdim=8,
                                                          tau=1.0)]
    mlps = [bu.moe(6, 2, 20, 3, 2, 1.0), bu.moe(8, 3, 12, 4, 3, 0.7), None, bu.moe(4, 1, 24, 1, 1, 2.0), bu.moe(6, 6, 8, 2, 2, 1.2)]
    return bu.config(layers, mlps, vocab=97, width=48, groups=4, taps=3)


def _cfg_b():
    layers = [bu.delta(2, 1, 24, 16, conv=3), bu.delta(1, 1, 8, 40, conv=5), bu.delta(5, 5, 6, 6, conv=4)]
    mlps = [bu.moe(5, 2, 16, 5, 3, 0.9), None, bu.moe(9, 4, 10, 3, 2, 1.5)]
    return bu.config(layers, mlps, vocab=53, width=30, eps=1e-6, groups=1, taps=2)


def _cfg_c():
    layers = [bu.parallel(2, 2, 12, 12, window=3, rot_dims=12, scale=0.5, r_heads=2, r_dim=16, r_vdim=10, tau=0.5),
              bu.parallel(8, 2, 10, 6, window=1000, rot_dims=6, scale=0.25, r_heads=4, r_dim=6, r_vdim=20, tau=6.0, left_scale=0.3,
                          right_scale=1.0)]
    mlps = [None, bu.moe(4, 2, 32, 2, 1, 1.0)]
    return bu.config(layers, mlps, vocab=61, width=40, groups=5, taps=4)


def _cfg_d():
    """The layers of ``a`` with routers that choose ALL their experts: nothing discrete is left, so bf16 runs can be
    held against the plain statement position by position (a close call of a router that falls the other way in bf16
    moves a position, and through the recurrent states the ones after it, by far more than rounding does)."""
    cfg = _cfg_a()
    for layer, size in zip(cfg["layers"], [(4, 20), (3, 16), None, (4, 24), (2, 8)]):
        if layer["mlp"] is not None:
            layer["mlp"] = bu.moe(size[0], size[0], size[1], 1, 1, 1.0)
    return cfg


def _cfg_e():
    """The least there can be: one layer without a feed-forward, convolutions of a single tap (nothing is carried)."""
    return bu.config([bu.delta(2, 2, 8, 8, conv=1)], [None], vocab=41, width=16, groups=2, taps=1)


_CASES = {"a": (_cfg_a, 11), "b": (_cfg_b, 12), "c": (_cfg_c, 13), "d": (_cfg_d, 14), "e": (_cfg_e, 15)}
FP32_TOL = 2e-4
BF16_TOL = 0.15         # five layers of ten normed sublayers: the worst position of a bf16 run stands near 0.10


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    out = {}
    for name, (make, seed) in _CASES.items():
        cfg = make()
        sd = bu.random_weights(cfg, seed, decay_rank=3 + seed % 4)
        path = bu.write_model(str(tmp_path_factory.mktemp("bogetar_" + name)), cfg, sd)
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
            cache[key] = bu.make_engine(models[name].path, dtype, **kw)
        return cache[key]
    return get


@pytest.mark.parametrize("name", sorted(_CASES))
def test_stream_after_every_layer(models, engines, name):
    m = models[name]
    engine = engines(name, "float32")
    model = engine.model_executor.driver_worker.model_runner.model
    toks = m.reqs["r4"]
    want = []
    oracle.logits(m.cfg, m.sd, toks, want, dtype=F64)
    model.keep_residuals = []
    try:
        bu.Replayer(engine, {"r4": toks}).run_alone("r4", [len(toks)])
        got = [r.cpu().double() for r in model.keep_residuals]
    finally:
        model.keep_residuals = None
    assert len(got) == len(want)
    for i, (a, b) in enumerate(zip(got, want)):
        assert (a - b).abs().max() < 1e-4 * b.abs().max(), f"layer {i} ({m.cfg['layers'][i]['type']})"


@pytest.mark.parametrize("name", sorted(_CASES))
def test_whole_prompts_match_the_plain_statement(models, engines, name):
    m = models[name]
    for rid, toks in m.reqs.items():
        got = bu.Replayer(engines(name, "float32"), {rid: toks}).run_alone(rid, [len(toks)])
        assert bu.row_error(got, m.want[rid]) < FP32_TOL, rid


@pytest.mark.parametrize("name", sorted(_CASES))
def test_decoding_token_by_token(models, engines, name):
    """Most of a prompt at once and then 45 (and 100) tokens one by one -- windows pass over decoded tokens --, and
    a sequence fed one token at a time from its very first."""
    m = models[name]
    for rid, first in (("r0", 25), ("r6", 50)):
        toks = m.reqs[rid]
        got = bu.Replayer(engines(name, "float32"), {rid: toks}).run_alone(rid, [first] + [1] * (len(toks) - first))
        assert bu.row_error(got, m.want[rid]) < FP32_TOL
    toks = m.reqs["r2"]
    got = bu.Replayer(engines(name, "float32"), {"r2": toks}).run_alone("r2", [1] * len(toks))
    assert bu.row_error(got, m.want["r2"]) < FP32_TOL


@pytest.mark.parametrize("name", sorted(_CASES))
@pytest.mark.parametrize("portions", [[2] * 35, [3, 2, 16, 1, 2, 7, 17, 2, 2, 18], [15, 1, 16, 17, 2, 19], [33, 31, 2, 4]])
def test_portions_of_prompts(models, engines, name, portions):
    m = models[name]
    toks = m.reqs["r0"]
    assert sum(portions) == len(toks)
    got = bu.Replayer(engines(name, "float32"), {"r0": toks}).run_alone("r0", portions)
    assert bu.row_error(got, m.want["r0"]) < FP32_TOL


@pytest.mark.parametrize("name,dtype,tol", [("a", "float32", FP32_TOL), ("b", "float32", FP32_TOL), ("c", "float32", FP32_TOL),
                                            ("d", "bfloat16", BF16_TOL)])
def test_mixed_batches_reuse_pages_and_slots(models, engines, name, dtype, tol):
    """Six unequal requests over three state slots and a pool of 9 pages: portions beside single tokens, requests
    that sit out steps, pages and slots handed on as requests end.  Every request must come out as it does alone."""
    m = models[name]
    reqs = {r: t for r, t in m.reqs.items() if r != "r6"}
    engine = engines(name, dtype, max_tokens=144, max_requests=3)
    rp = bu.Replayer(engine, reqs)
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
        if dtype == "bfloat16":                                 # the worst position of a bf16 run is not a stable number
            assert bu.share_within(rp.result(rid), m.want[rid], tol) >= 0.9 and bu.row_error(rp.result(rid), m.want[rid]) < 3 * tol, rid
        else:
            assert bu.row_error(rp.result(rid), m.want[rid]) < tol, rid
    assert engine.scheduler.block_manager.get_num_free_gpu_blocks() == free_before
    assert engine.scheduler.state_slots.num_free() == 3


def test_bfloat16_is_close_and_does_not_depend_on_the_cut(models, engines):
    m = models["d"]
    toks = m.reqs["r0"]
    whole = bu.Replayer(engines("d", "bfloat16"), {"r0": toks}).run_alone("r0", [len(toks)])
    cut = bu.Replayer(engines("d", "bfloat16"), {"r0": toks}).run_alone("r0", [2, 3, 16, 1, 1, 30, 17])
    assert bu.row_error(whole, m.want["r0"]) < BF16_TOL
    assert bu.row_error(cut, m.want["r0"]) < BF16_TOL
    assert bu.row_error(cut, whole) < 0.05
    # with routers that choose (model a) most positions still agree; the others follow a close call
    m = models["a"]
    whole = bu.Replayer(engines("a", "bfloat16"), {"r0": m.reqs["r0"]}).run_alone("r0", [len(m.reqs["r0"])])
    assert bu.share_within(whole, m.want["r0"], BF16_TOL) >= 0.8


@pytest.mark.parametrize("name", sorted(_CASES))
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
    m = models["c"]
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
        assert bu.row_error(got, torch.stack(rows)) < FP32_TOL, step

"""Throughput of a Nepevik (or Lapilorn, Lalasun or Bogetar) stack beside a Llama stack of the same width, depth and active feed-forward size
(random weights), and every mixer kernel beside the like kernel of the Llama path with their distances from
the roofline.  ``bench.py --mixers`` prints the result as one JSON line.

Engine level: PREFILL = prompt tokens per second from the first step to the last prompt's first token;
DECODE = generated tokens per second over a run of pure decode steps at a fixed batch.  Both go through
``LLMEngine.step`` (scheduler, block tables, sampler), so host time counts.

Kernel level: HIP-event time per launch; ``roof`` = the larger of (algorithmic bytes / HBM peak) and
(flops / the unit's peak) divided by the measured time: 1.0 would be the roofline.  Matrix work on MFMA is
priced at the dense bf16 peak, everything else at the fp32 vector peak.
"""
import time
from typing import Dict, List

import torch

HBM_BPS = 8.0e12
MFMA_BF16 = 2.5e15
VALU_F32 = 157.0e12          # 256 CUs x 4 SIMDs x 16 lanes x 2 (fma) x 2 (packed pairs) x 2.4 GHz: the published vector peak


def _sync() -> None:
    torch.cuda.synchronize()


def engine_throughput(model: str, prompt_len: int = 2048, prompts: int = 8, decode_batch: int = 64,
                      decode_prompt: int = 512, decode_steps: int = 48, budget: int = 4096) -> Dict[str, float]:
    from ..engine.arg_utils import EngineArgs
    from ..engine.llm_engine import LLMEngine
    from ..sampling_params import SamplingParams
    block = 16
    need = max(prompts * (prompt_len + block), decode_batch * (decode_prompt + decode_steps + 2 * block))
    engine = LLMEngine.from_engine_args(EngineArgs(
        model=model, dtype="bfloat16", block_size=block, max_model_len=max(prompt_len, decode_prompt + decode_steps) + block,
        max_num_seqs=max(decode_batch, prompts), max_num_batched_tokens=max(budget, prompt_len + block),
        num_gpu_blocks_override=need // block + 64, swap_space=0))
    vocab = engine.model_config.get_vocab_size()
    gen = torch.Generator().manual_seed(0)

    def tokens(n):
        return torch.randint(0, vocab, (n,), generator=gen).tolist()

    def drain():
        while engine.has_unfinished_requests():
            engine.step()

    out = {}
    for rep in range(2):                                   # the first pass warms libraries and allocators up
        for i in range(prompts):
            engine.add_request(f"p{rep}-{i}", None, SamplingParams(temperature=0.0, max_tokens=1, ignore_eos=True),
                               prompt_token_ids=tokens(prompt_len))
        _sync()
        t0 = time.perf_counter()
        drain()
        _sync()
        out["prefill_tok_s"] = prompts * prompt_len / (time.perf_counter() - t0)
    for i in range(decode_batch):
        engine.add_request(f"d{i}", None, SamplingParams(temperature=0.0, max_tokens=decode_steps + 8, ignore_eos=True),
                           prompt_token_ids=tokens(decode_prompt))
    # run until every request has its first token and a few decode steps have gone by
    while any(len(g.get_seqs()[0].get_output_token_ids()) < 4 for g in engine.scheduler.running) or engine.scheduler.waiting:
        engine.step()
    _sync()
    t0 = time.perf_counter()
    for _ in range(decode_steps - 8):
        engine.step()
    _sync()
    out["decode_tok_s"] = decode_batch * (decode_steps - 8) / (time.perf_counter() - t0)
    out["decode_ms_per_step"] = 1e3 * decode_batch / out["decode_tok_s"]
    drain()
    del engine
    torch.cuda.empty_cache()
    return out


def _time(fn, iters: int = 20, warmup: int = 3) -> float:
    for _ in range(warmup):
        fn()
    _sync()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(iters):
        fn()
    b.record()
    _sync()
    return a.elapsed_time(b) / iters * 1e-3


def _row(name: str, phase: str, t: float, nbytes: float, flops: float, peak: float, like: str = "") -> dict:
    floor = max(nbytes / HBM_BPS, flops / peak)
    return {"kernel": name, "phase": phase, "us": round(t * 1e6, 1), "GBps": round(nbytes / t / 1e9, 1),
            "TFLOPs": round(flops / t / 1e12, 2), "roof": round(floor / t, 4), "like": like}


def _ragged(seqs, dev):
    """[(ctx, new tokens, slot, table)] -> an object with the ragged layout's tensors."""
    from types import SimpleNamespace
    q_start, token_seq = [0], []
    for i, (_, n, _, _) in enumerate(seqs):
        q_start.append(q_start[-1] + n)
        token_seq += [i] * n
    width = max(max(len(s[3]) for s in seqs), 1)
    tables = torch.zeros(len(seqs), width, dtype=torch.int32)
    for i, s in enumerate(seqs):
        tables[i, :len(s[3])] = torch.tensor(s[3], dtype=torch.int32)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=dev)        # noqa: E731
    return SimpleNamespace(q_start=i32(q_start), ctx_len=i32([s[0] for s in seqs]), token_seq=i32(token_seq),
                           state_slot=i32([s[2] for s in seqs]), block_tables=tables.to(dev), num_seqs=len(seqs),
                           max_query_len=max(s[1] for s in seqs), max_pages_used=width,
                           max_page_id=int(tables.max()), max_state_slot=max(s[2] for s in seqs))


@torch.inference_mode()
def kernel_table(width: int = 2048, heads: int = 16, kv_heads: int = 4, window: int = 1024, keep: int = 16,
                 prefill_rows: int = 4096, decode_seqs: int = 64, decode_ctx: int = 2048, experts: int = 32,
                 top: int = 2, ff: int = 1024) -> List[dict]:
    from .. import _C
    dev, bf = torch.device("cuda"), torch.bfloat16
    d = width // heads
    page = 16
    rows: List[dict] = []
    scale = d ** -0.5

    # ------------------------------------------------------------------ attention
    for phase, seqs in (("prefill", [(0, prefill_rows // 2, 0, None), (0, prefill_rows // 2, 1, None)]),
                        ("decode", [(decode_ctx, 1, i, None) for i in range(decode_seqs)])):
        total_pages, laid = 0, []
        for ctx, n, slot, _ in seqs:
            pages = -(-(ctx + n) // page)
            laid.append((ctx, n, slot, list(range(total_pages, total_pages + pages))))
            total_pages += pages
        batch = _ragged(laid, dev)
        T = sum(s[1] for s in laid)
        kc = torch.randn(total_pages, page, kv_heads * d, device=dev).to(bf)
        vc = torch.randn(total_pages, page, kv_heads * d, device=dev).to(bf)
        q = torch.randn(T, heads * d, device=dev)
        talk = torch.eye(heads, device=dev) + 0.1 * torch.randn(heads, heads, device=dev)
        out = torch.empty(T, heads * d, dtype=bf, device=dev)
        t = _time(lambda: _C.mixer_ops.window_attention(out, q, kc, vc, talk, batch, heads, kv_heads, d, d, scale, window,
                                                        keep))
        pairs = sum(min(c + i + 1, window + keep) for c, n, _, _ in laid for i in range(n))      # (query, key) pairs
        keys = sum(min(c + n, (window + keep) if phase == "decode" else c + n) for c, n, _, _ in laid)
        flops = 2.0 * pairs * heads * (d + kv_heads * d)
        nbytes = keys * kv_heads * d * 2 * 2 + T * heads * d * (4 + 2)
        rows.append(_row("window_attention (talking heads)", phase, t, nbytes, flops,
                         VALU_F32))            # its weights stay fp32: the bf16 matrix path is closed to it
        # the Llama path's kernel at the same head geometry
        if phase == "prefill":
            qh = torch.randn(T, heads, d, device=dev).to(bf)
            kh = torch.randn(T, kv_heads, d, device=dev).to(bf)
            vh = torch.randn(T, kv_heads, d, device=dev).to(bf)
            oh = torch.empty_like(qh)
            starts = torch.tensor([0, T // 2], dtype=torch.int32, device=dev)
            lens = torch.tensor([T // 2, T // 2], dtype=torch.int32, device=dev)
            t2 = _time(lambda: _C.ops.prefill_attention(oh, qh, kh, vh, starts, lens, T // 2, scale, None, window))
            pairs2 = sum(min(i + 1, window) for i in range(T // 2)) * 2
            rows.append(_row("prefill_attention (sliding window)", phase, t2, T * (heads + 2 * kv_heads) * d * 2 + T * heads * d * 2,
                             4.0 * pairs2 * heads * d, MFMA_BF16, like="window_attention"))
        else:
            x = 8
            nb = decode_seqs * (-(-window // page)) + 1
            kc2 = torch.randn(nb, kv_heads, d // x, page, x, device=dev).to(bf)
            vc2 = torch.randn(nb, kv_heads, d, page, device=dev).to(bf)
            bt = torch.randperm(nb - 1, device=dev).to(torch.int32).view(decode_seqs, -1).contiguous()
            cl = torch.full((decode_seqs,), window, dtype=torch.int32, device=dev)
            qh = torch.randn(decode_seqs, heads, d, device=dev).to(bf)
            oh = torch.empty_like(qh)
            t2 = _time(lambda: _C.ops.paged_attention_v1(oh, qh, kc2, vc2, kv_heads, scale, bt, cl, page, window, None, "auto"))
            rows.append(_row("paged_attention_v1 (window's worth of context)", phase, t2,
                             decode_seqs * window * kv_heads * d * 2 * 2 + 2 * decode_seqs * heads * d * 2,
                             4.0 * decode_seqs * window * heads * d, VALU_F32, like="window_attention"))

    # ------------------------------------------------------------------ delta rules, convolution, gates
    for phase, seqs in (("prefill", [(0, prefill_rows // 2, 0, []), (0, prefill_rows // 2, 1, [])]),
                        ("decode", [(decode_ctx, 1, i, []) for i in range(decode_seqs)])):
        batch = _ragged(seqs, dev)
        T, B = sum(s[1] for s in seqs), len(seqs)
        slots = max(B, 2)
        # channel-decay rule: heads x [d, d]
        qkv = torch.randn(T, 3 * heads * d, device=dev)
        beta = torch.randn(T, heads, device=dev).to(bf)
        decay = torch.randn(T, heads * d, device=dev).to(bf)
        state = torch.zeros(slots, heads, d, d, device=dev)
        o = torch.empty(T, heads * d, device=dev)
        dt_bias, a_log = torch.zeros(heads * d, device=dev), torch.zeros(heads, device=dev)
        t = _time(lambda: _C.mixer_ops.channel_delta(o, qkv, beta, decay, dt_bias, a_log, state, batch, heads, heads, d, d))
        nbytes = T * (3 * heads * d * 4 + heads * d * 2 + heads * d * 4) + 2 * B * heads * d * d * 4
        rows.append(_row("channel_delta", phase, t, nbytes, 8.0 * T * heads * d * d, VALU_F32))
        # general rule: 2 * heads x [d / 2, d / 2]
        h2, d2 = 2 * heads, d // 2
        proj = torch.randn(T, 5 * h2 * d2, device=dev).to(bf)
        n = h2 * d2
        wpre = torch.randn(T, n, device=dev).to(bf)
        state2 = torch.zeros(slots, h2, d2, d2, device=dev)
        o2 = torch.empty(T, n, device=dev)
        zeros = torch.zeros(n, device=dev)
        t = _time(lambda: _C.mixer_ops.general_delta(o2, proj[:, :n], proj[:, n:2 * n], proj[:, 2 * n:3 * n], wpre, zeros,
                                                     proj[:, 4 * n:], zeros, state2, batch, h2, d2))
        rows.append(_row("general_delta", phase, t, T * n * (5 * 2 + 4) + 2 * B * h2 * d2 * d2 * 4, 9.0 * T * h2 * d2 * d2,
                         VALU_F32))
        # short convolution over q | k | v channels
        ch = 3 * heads * d
        xin = torch.randn(T, ch, device=dev).to(bf)
        taps = torch.randn(ch, 4, device=dev)
        cstate = torch.zeros(slots, 3, ch, device=dev)
        cout = torch.empty(T, ch, device=dev)
        t = _time(lambda: _C.mixer_ops.short_conv(cout, xin, taps, cstate, batch))
        rows.append(_row("short_conv (+ state advance)", phase, t, T * ch * (2 + 4) + 2 * B * 3 * ch * 4, 8.0 * T * ch, VALU_F32))
        # per-head norm and gate
        gate = torch.randn(T, heads * d, device=dev).to(bf)
        wn = torch.ones(d, device=dev)
        g_out = torch.empty(T, heads * d, dtype=bf, device=dev)
        t = _time(lambda: _C.mixer_ops.head_norm_gate(g_out, o, gate, wn, False, 1e-6, heads, d))
        rows.append(_row("head_norm_gate", phase, t, T * heads * d * (4 + 2 + 2), 6.0 * T * heads * d, VALU_F32))
        # norm of a sublayer's output added to the fp32 stream  /  Llama's fused add + norm
        res = torch.randn(T, width, device=dev)
        y = torch.randn(T, width, device=dev).to(bf)
        cast = torch.empty(T, width, dtype=bf, device=dev)
        gain = torch.ones(1, device=dev)
        t = _time(lambda: _C.mixer_ops.scalar_norm_add(res, y, gain, 1e-6, cast))
        rows.append(_row("scalar_norm_add (fp32 stream)", phase, t, T * width * (2 + 4 + 4 + 2), 4.0 * T * width, VALU_F32))
        xr, rr, wr = y.clone(), y.clone(), torch.ones(width, dtype=bf, device=dev)
        t = _time(lambda: _C.ops.fused_add_rms_norm(xr, rr, wr, 1e-6))
        rows.append(_row("fused_add_rms_norm (bf16 stream)", phase, t, T * width * 2 * 4, 4.0 * T * width, VALU_F32,
                         like="scalar_norm_add"))
        # experts against a dense feed-forward of the same active size
        hin = torch.randn(T, width, device=dev).to(bf)
        up = torch.randn(experts, ff, width, device=dev).to(bf) * 0.02
        down = torch.randn(experts, width, ff, device=dev).to(bf) * 0.02
        choice = torch.rand(T, experts, device=dev).argsort(1)[:, :top].reshape(-1)
        order = torch.sort(choice, stable=True).indices.to(torch.int32)
        start = torch.zeros(experts + 1, dtype=torch.int32, device=dev)
        start[1:] = torch.cumsum(torch.bincount(choice, minlength=experts), 0)
        eo = torch.zeros(T, width, device=dev)
        t = _time(lambda: _C.mixer_ops.expert_ffn(eo, hin, up, down, order, start, top, 1.0 / top))
        flops = 4.0 * T * top * ff * width
        touched = min(experts, T * top)
        nbytes = touched * 2 * ff * width * 2 + T * width * (2 + 4) + T * top * ff * 2 * 2
        rows.append(_row("expert_ffn (grouped, gelu)", phase, t, nbytes, flops, MFMA_BF16))
        w1 = torch.randn(top * ff, width, device=dev).to(bf) * 0.02
        w2 = torch.randn(width, top * ff, device=dev).to(bf) * 0.02
        t = _time(lambda: torch.nn.functional.linear(torch.nn.functional.gelu(torch.nn.functional.linear(hin, w1)), w2))
        rows.append(_row("dense feed-forward of the same active size (library GEMMs)", phase, t,
                         2 * top * ff * width * 2 + T * width * 4 + T * top * ff * 4, flops, MFMA_BF16, like="expert_ffn"))
    return rows


@torch.inference_mode()
def kernel_table_lapilorn(width: int = 2048, heads: int = 16, kv_heads: int = 4, prefill_rows: int = 4096,
                          decode_seqs: int = 64, decode_ctx: int = 2048, experts: int = 32, top: int = 2,
                          ff: int = 1024) -> List[dict]:
    """The kernels of the Lapilorn layers beside the like kernels of the Llama path (or, for the recurrence, of the
    delta-rule layers).  fp32 matrix work (scores, softmax weights and states must stay fp32) is priced at the fp32
    matrix peak, which equals the fp32 vector peak on this GPU."""
    from .. import _C
    dev, bf = torch.device("cuda"), torch.bfloat16
    d = width // heads
    page = 16
    rows: List[dict] = []
    scale = d ** -0.5
    for phase, seqs in (("prefill", [(0, prefill_rows // 2, 0, None), (0, prefill_rows // 2, 1, None)]),
                        ("decode", [(decode_ctx, 1, i, None) for i in range(decode_seqs)])):
        total_pages, laid = 0, []
        for ctx, n, slot, _ in seqs:
            pages = -(-(ctx + n) // page)
            laid.append((ctx, n, slot, list(range(total_pages, total_pages + pages))))
            total_pages += pages
        batch = _ragged(laid, dev)
        T, B = sum(s[1] for s in laid), len(laid)
        # ---------------------------------------------------------------- attention
        kc = torch.randn(total_pages, page, kv_heads * d, device=dev).to(bf)
        vc = torch.randn(total_pages, page, kv_heads * d, device=dev).to(bf)
        q = torch.randn(T, heads * d, device=dev)
        gate = torch.randn(T, heads * d, device=dev).to(bf)
        out = torch.empty(T, heads * d, dtype=bf, device=dev)
        t = _time(lambda: _C.mixer_ops.capped_attention(out, q, kc, vc, gate, batch, heads, kv_heads, d, d, scale, 30.0, 0))
        pairs = sum(c + i + 1 for c, n, _, _ in laid for i in range(n))
        keys = sum(c + n for c, n, _, _ in laid)
        rows.append(_row("capped_attention (fp32 matrix cores, gate fused)", phase, t,
                         keys * kv_heads * d * 2 * 2 + T * heads * d * (4 + 2 + 2), 4.0 * pairs * heads * d, VALU_F32))
        if phase == "prefill":
            qh = torch.randn(T, heads, d, device=dev).to(bf)
            kh = torch.randn(T, kv_heads, d, device=dev).to(bf)
            vh = torch.randn(T, kv_heads, d, device=dev).to(bf)
            oh = torch.empty_like(qh)
            starts = torch.tensor([0, T // 2], dtype=torch.int32, device=dev)
            lens = torch.tensor([T // 2, T // 2], dtype=torch.int32, device=dev)
            t2 = _time(lambda: _C.ops.prefill_attention(oh, qh, kh, vh, starts, lens, T // 2, scale, None, None))
            rows.append(_row("Llama prefill_attention (bf16 matrix cores)", phase, t2,
                             T * (heads + 2 * kv_heads) * d * 2 + T * heads * d * 2, 4.0 * pairs * heads * d, MFMA_BF16,
                             like="capped_attention"))
        else:
            x = 8
            per_seq = -(-(decode_ctx + 1) // page)
            nb = decode_seqs * per_seq + 1
            kc2 = torch.randn(nb, kv_heads, d // x, page, x, device=dev).to(bf)
            vc2 = torch.randn(nb, kv_heads, d, page, device=dev).to(bf)
            bt = torch.randperm(nb - 1, device=dev).to(torch.int32).view(decode_seqs, -1).contiguous()
            cl = torch.full((decode_seqs,), decode_ctx + 1, dtype=torch.int32, device=dev)
            qh = torch.randn(decode_seqs, heads, d, device=dev).to(bf)
            oh = torch.empty_like(qh)
            t2 = _time(lambda: _C.ops.paged_attention_v1(oh, qh, kc2, vc2, kv_heads, scale, bt, cl, page, decode_ctx + 1,
                                                         None, "auto"))
            rows.append(_row("Llama paged_attention_v1", phase, t2,
                             decode_seqs * (decode_ctx + 1) * kv_heads * d * 2 * 2 + 2 * decode_seqs * heads * d * 2,
                             4.0 * decode_seqs * (decode_ctx + 1) * heads * d, VALU_F32, like="capped_attention"))
        # ---------------------------------------------------------------- rotation + cache write
        proj = torch.randn(T, (heads + 2 * kv_heads) * d, device=dev).to(bf)
        pos = torch.cat([torch.arange(c, c + n) for c, n, _, _ in laid]).to(dev)
        slots = torch.cat([torch.tensor([tb[p // page] * page + p % page for p in range(c, c + n)])
                           for c, n, _, tb in laid]).to(dev)
        inv = torch.rand(d // 4, device=dev)
        q32 = torch.empty(T, heads * d, device=dev)
        t = _time(lambda: _C.mixer_ops.rope_cache(q32, proj[:, :heads * d], proj[:, heads * d:(heads + kv_heads) * d],
                                                  proj[:, (heads + kv_heads) * d:], pos, inv, heads, kv_heads, d, d, kc, vc,
                                                  slots))
        rows.append(_row("rope_cache (fp32 angles, fp32 queries out)", phase, t,
                         T * ((heads + 2 * kv_heads) * d * 2 + heads * d * 4 + 2 * kv_heads * d * 2), 6.0 * T * heads * d,
                         VALU_F32))
        # ---------------------------------------------------------------- lightning / delta rule
        lseqs = [(c, n, i, []) for i, (c, n, _, _) in enumerate(laid)]
        lbatch = _ragged(lseqs, dev)
        lproj = torch.randn(T, 3 * heads * d, device=dev).to(bf)
        state = torch.zeros(max(B, 2), heads, d, d, device=dev)
        decay = torch.full((heads,), 0.97, device=dev)
        lo = torch.empty(T, heads * d, device=dev)
        t = _time(lambda: _C.mixer_ops.lightning(lo, lproj[:, :heads * d], lproj[:, heads * d:2 * heads * d],
                                                 lproj[:, 2 * heads * d:], decay, state, lbatch, heads, d, d))
        chunk = 32
        lflops = T * heads * (2.0 * chunk * d + 2.0 * chunk * d + 4.0 * d * d)      # in-chunk scores and sums, state in and out
        lbytes = T * heads * d * (3 * 2 + 4) + 2 * B * heads * d * d * 4
        rows.append(_row("lightning (chunks of 32 on fp32 matrix cores)", phase, t, lbytes, lflops, VALU_F32))
        qkv = torch.randn(T, 3 * heads * d, device=dev)
        beta = torch.randn(T, heads, device=dev).to(bf)
        dpre = torch.randn(T, heads * d, device=dev).to(bf)
        o = torch.empty(T, heads * d, device=dev)
        dt_bias, a_log = torch.zeros(heads * d, device=dev), torch.zeros(heads, device=dev)
        t2 = _time(lambda: _C.mixer_ops.channel_delta(o, qkv, beta, dpre, dt_bias, a_log, state, lbatch, heads, heads, d, d))
        rows.append(_row("Nepevik channel_delta (token by token)", phase, t2,
                         T * (3 * heads * d * 4 + heads * d * 2 + heads * d * 4) + 2 * B * heads * d * d * 4,
                         8.0 * T * heads * d * d, VALU_F32, like="lightning"))
        # ---------------------------------------------------------------- whole-heads norm and gate
        gated = torch.empty(T, heads * d, dtype=bf, device=dev)
        wn = torch.ones(heads * d, device=dev)
        t = _time(lambda: _C.mixer_ops.head_norm_gate(gated, lo, gate, wn, True, 1e-6, 1, heads * d))
        rows.append(_row("head_norm_gate (one norm over all heads)", phase, t, T * heads * d * (4 + 2 + 2), 6.0 * T * heads * d,
                         VALU_F32))
        # ---------------------------------------------------------------- residual add + next norm
        res = torch.randn(T, width, device=dev)
        a = torch.randn(T, width, device=dev).to(bf)
        b2 = torch.randn(T, width, device=dev).to(bf)
        c32 = torch.randn(T, width, device=dev)
        hout = torch.empty(T, width, dtype=bf, device=dev)
        wgt = torch.zeros(width, device=dev)
        t = _time(lambda: _C.mixer_ops.stream_add_norm(res, wgt, 1.0, 1e-6, hout, a, b2, None))
        rows.append(_row("stream_add_norm (fp32 stream, two addends)", phase, t, T * width * (4 + 4 + 2 + 2 + 2), 6.0 * T * width,
                         VALU_F32))
        t = _time(lambda: _C.mixer_ops.stream_add_norm(res, wgt, 1.0, 1e-6, hout, a, b2, c32))
        rows.append(_row("stream_add_norm (three addends, one fp32)", phase, t, T * width * (4 + 4 + 2 + 2 + 4 + 2), 7.0 * T * width,
                         VALU_F32))
        xr, rr, wr = a.clone(), a.clone(), torch.ones(width, dtype=bf, device=dev)
        t2 = _time(lambda: _C.ops.fused_add_rms_norm(xr, rr, wr, 1e-6))
        rows.append(_row("Llama fused_add_rms_norm (bf16 stream)", phase, t2, T * width * 2 * 4, 4.0 * T * width, VALU_F32,
                         like="stream_add_norm"))
        # ---------------------------------------------------------------- gated activation
        dff = (11 * ff) // 4
        gu = torch.randn(T, 2 * dff, device=dev).to(bf)
        act = torch.empty(T, dff, dtype=bf, device=dev)
        t = _time(lambda: _C.mixer_ops.clamped_glu(act, gu, 1.702, 7.0, 1.0))
        rows.append(_row("clamped_glu", phase, t, T * dff * 3 * 2, 8.0 * T * dff, VALU_F32))
        t2 = _time(lambda: _C.ops.silu_and_mul(act, gu))
        rows.append(_row("Llama silu_and_mul", phase, t2, T * dff * 3 * 2, 5.0 * T * dff, VALU_F32, like="clamped_glu"))
        # ---------------------------------------------------------------- router and experts
        hin = torch.randn(T, width, device=dev).to(bf)
        router = torch.randn(experts, width, device=dev) * width ** -0.5
        corr = torch.randn(experts, device=dev) * 0.1
        t = _time(lambda: _C.mixer_ops.group_router(torch.matmul(hin.float(), router.t()), corr, top, 4, 2, 2.5))
        rows.append(_row("router: fp32 GEMM + group_router", phase, t, T * width * 2 + experts * width * 4 + T * top * 8,
                         2.0 * T * experts * width, VALU_F32))
        chosen, weights = _C.mixer_ops.group_router(torch.matmul(hin.float(), router.t()), corr, top, 4, 2, 2.5)
        from ..model_executor.layers.moe import group_pairs_by_expert
        order, start = group_pairs_by_expert(chosen, experts)
        up = torch.randn(experts, ff, width, device=dev).to(bf) * 0.02
        down = torch.randn(experts, width, ff, device=dev).to(bf) * 0.02
        eo = torch.zeros(T, width, device=dev)
        t = _time(lambda: _C.mixer_ops.expert_ffn(eo, hin, up, down, order, start, top, 1.0,
                                                  activation=_C.mixer_ops.ACT_RELU2, pair_weight=weights))
        flops = 4.0 * T * top * ff * width
        touched = min(experts, T * top)
        rows.append(_row("expert_ffn (grouped, relu^2, weighted)", phase, t,
                         touched * 2 * ff * width * 2 + T * width * (2 + 4) + T * top * ff * 2 * 2, flops, MFMA_BF16))
        w1 = torch.randn(top * ff, width, device=dev).to(bf) * 0.02
        w2 = torch.randn(width, top * ff, device=dev).to(bf) * 0.02
        t2 = _time(lambda: torch.nn.functional.linear(torch.nn.functional.gelu(torch.nn.functional.linear(hin, w1)), w2))
        rows.append(_row("dense feed-forward of the same active size (library GEMMs)", phase, t2,
                         2 * top * ff * width * 2 + T * width * 4 + T * top * ff * 4, flops, MFMA_BF16, like="expert_ffn"))
    return rows


@torch.inference_mode()
def kernel_table_lalasun(width: int = 2048, heads: int = 16, kv_heads: int = 4, prefill_rows: int = 4096,
                         decode_seqs: int = 64, decode_ctx: int = 2047, rank: int = 192, rot: int = 64, span: int = 1024,
                         ff: int = 4224, depth: int = 6) -> List[dict]:
    """The kernels of the Lalasun layers beside their like: the attention kernel with a chunk mask and a sink, and
    over a shared latent, beside the same kernel as Lapilorn calls it (plain causal, grouped heads); the recurrence
    with a decay per key channel beside the one with a decay per head; the gated stream step beside the fused add +
    RMS norm; PolyNorm beside the clamped gated unit."""
    from .. import _C
    dev, bf = torch.device("cuda"), torch.bfloat16
    d = width // heads
    page = 16
    rows: List[dict] = []
    scale = d ** -0.5
    for phase, seqs in (("prefill", [(0, prefill_rows // 2, 0, None), (0, prefill_rows // 2, 1, None)]),
                        ("decode", [(decode_ctx, 1, i, None) for i in range(decode_seqs)])):
        total_pages, laid = 0, []
        for ctx, n, slot, _ in seqs:
            pages = -(-(ctx + n) // page)
            laid.append((ctx, n, slot, list(range(total_pages, total_pages + pages))))
            total_pages += pages
        batch = _ragged(laid, dev)
        T, B = sum(s[1] for s in laid), len(laid)

        def seen(limit_kind):
            """(query, key) pairs and distinct keys read under a mask."""
            pairs = keys = 0
            for c, n, _, _ in laid:
                for i in range(c, c + n):
                    lo = 0 if limit_kind == "all" else i // span * span if limit_kind == "chunk" else max(0, i - span + 1)
                    pairs += i - lo + 1
                first = c if n == 1 else 0
                lo = 0 if limit_kind == "all" else first // span * span if limit_kind == "chunk" else max(0, first - span + 1)
                keys += c + n - lo
            return pairs, keys
        # ---------------------------------------------------------------- attention, grouped heads
        kc = torch.randn(total_pages, page, kv_heads * d, device=dev).to(bf)
        vc = torch.randn(total_pages, page, kv_heads * d, device=dev).to(bf)
        q = torch.randn(T, heads * d, device=dev)
        out = torch.empty(T, heads * d, dtype=bf, device=dev)
        for name, kind, kw, like in (("masked attention (chunks of %d, sink)" % span, "chunk", dict(chunk=span, sink=True), ""),
                                     ("capped_attention as Lapilorn runs it (causal, no cap)", "all", {}, "masked attention")):
            t = _time(lambda: _C.mixer_ops.capped_attention(out, q, kc, vc, None, batch, heads, kv_heads, d, d, scale, 0.0, 0, **kw))
            pairs, keys = seen(kind)
            rows.append(_row(name, phase, t, keys * kv_heads * d * 2 * 2 + T * heads * d * (4 + 2), 4.0 * pairs * heads * d,
                             VALU_F32, like=like))
        # ---------------------------------------------------------------- attention over a shared latent
        row = rank + rot
        lc = torch.randn(total_pages, page, row, device=dev).to(bf)
        ql = torch.randn(T, heads * row, device=dev)
        lout = torch.empty(T, heads * rank, dtype=bf, device=dev)
        t = _time(lambda: _C.mixer_ops.capped_attention(lout, ql, lc, None, None, batch, heads, 1, row, rank, scale, 0.0, span))
        pairs, keys = seen("window")
        rows.append(_row("latent attention (one %d-wide row per token, window %d)" % (row, span), phase, t,
                         keys * row * 2 + T * heads * (row * 4 + rank * 2), 2.0 * pairs * heads * (row + rank), VALU_F32,
                         like="capped_attention"))
        # ---------------------------------------------------------------- rotation and cache writes
        pos = torch.cat([torch.arange(c, c + n) for c, n, _, _ in laid]).to(dev)
        slots = torch.cat([torch.tensor([tb[p // page] * page + p % page for p in range(c, c + n)])
                           for c, n, _, tb in laid]).to(dev)
        proj = torch.randn(T, (heads + 2 * kv_heads) * d, device=dev).to(bf)
        inv = torch.rand(d // 2, device=dev)
        q32 = torch.empty(T, heads * d, device=dev)
        for name, halves, like in (("rope_cache, pairs (i, i + d/2)", True, ""), ("rope_cache, neighbouring pairs", False, "rope_cache")):
            t = _time(lambda: _C.mixer_ops.rope_cache(q32, proj[:, :heads * d], proj[:, heads * d:(heads + kv_heads) * d],
                                                      proj[:, (heads + kv_heads) * d:], pos, inv, heads, kv_heads, d, d, kc,
                                                      vc, slots, halves))
            rows.append(_row(name, phase, t, T * ((heads + 2 * kv_heads) * d * 2 + heads * d * 4 + 2 * kv_heads * d * 2),
                             6.0 * T * heads * d, VALU_F32, like=like))
        q_lat = torch.randn(heads, T, rank, device=dev).to(bf)
        lproj = torch.randn(T, heads * (d // 2 + rot) + row, device=dev).to(bf)
        qrot = lproj[:, :heads * (d // 2 + rot)].unflatten(1, (heads, d // 2 + rot))[:, :, d // 2:]
        wl = torch.ones(rank, device=dev)
        invl = torch.rand(rot // 2, device=dev)
        t = _time(lambda: _C.mixer_ops.latent_rope_cache(ql, q_lat.transpose(0, 1), qrot, lproj[:, heads * (d // 2 + rot):], wl,
                                                         1e-6, pos, invl, lc, slots))
        rows.append(_row("latent_rope_cache (latent norm, rotation, query layout)", phase, t,
                         T * (heads * (rank + rot) * (2 + 4) + row * 2 * 2), 6.0 * T * heads * rot, VALU_F32, like="rope_cache"))
        # ---------------------------------------------------------------- recurrences
        dk = d // 2
        lseqs = [(c, n, i, []) for i, (c, n, _, _) in enumerate(laid)]
        lbatch = _ragged(lseqs, dev)
        gproj = torch.randn(T, heads * (2 * dk + d), device=dev).to(bf)
        zpre = torch.randn(T, heads * dk, device=dev).to(bf)
        zbias = torch.full((heads * dk,), 2.0, device=dev)
        state = torch.zeros(max(B, 2), heads, dk, d, device=dev)
        go = torch.empty(T, heads * d, device=dev)
        t = _time(lambda: _C.mixer_ops.gla(go, gproj[:, :heads * dk], gproj[:, heads * dk:2 * heads * dk],
                                           gproj[:, 2 * heads * dk:], zpre, zbias, 8.0, dk ** -0.5, state, lbatch, heads, dk, d))
        chunk = 32
        gflops = T * heads * (2.0 * chunk * dk + 2.0 * chunk * d + 4.0 * dk * d)
        gbytes = T * heads * ((3 * dk + d) * 2 + d * 4) + 2 * B * heads * dk * d * 4
        rows.append(_row("gla (decay per key channel)", phase, t, gbytes, gflops, VALU_F32))
        decay = torch.full((heads,), 0.97, device=dev)
        t2 = _time(lambda: _C.mixer_ops.lightning(go, gproj[:, :heads * dk], gproj[:, heads * dk:2 * heads * dk],
                                                  gproj[:, 2 * heads * dk:], decay, state, lbatch, heads, dk, d))
        rows.append(_row("Lapilorn lightning (decay per head), same sizes", phase, t2,
                         T * heads * ((2 * dk + d) * 2 + d * 4) + 2 * B * heads * dk * d * 4, gflops, VALU_F32, like="gla"))
        gate = torch.randn(T, heads * d, device=dev).to(bf)
        gated = torch.empty(T, heads * d, dtype=bf, device=dev)
        wn = torch.ones(d, device=dev)
        t = _time(lambda: _C.mixer_ops.head_norm_gate(gated, go, gate, wn, False, 1e-6, heads, d, gate_silu=True))
        rows.append(_row("head_norm_gate (per head, silu gate)", phase, t, T * heads * d * (4 + 2 + 2), 8.0 * T * heads * d, VALU_F32))
        up = torch.randn(heads, T, d, device=dev).to(bf)
        t = _time(lambda: _C.mixer_ops.gate_mul(gated, up.transpose(0, 1), gate))
        rows.append(_row("gate_mul (heads of a batched product, sigmoid gate)", phase, t, T * heads * d * 2 * 3, 4.0 * T * heads * d,
                         VALU_F32))
        # ---------------------------------------------------------------- stream steps
        stream = torch.randn(T, width, device=dev)
        y = torch.randn(T, 2 * width, device=dev).to(bf)
        hist = torch.randn(depth, T, width, device=dev)
        dw = torch.rand(depth, device=dev)
        norm = (torch.full((1,), 0.5, device=dev), torch.ones(width, device=dev), torch.zeros(width, device=dev))
        hout = torch.empty(T, width, dtype=bf, device=dev)
        t = _time(lambda: _C.mixer_ops.gated_stream_step(stream, y[:, :width], y[:, width:], 0.5, None, None, norm, hout))
        rows.append(_row("gated_stream_step (gated add + tanh norm)", phase, t, T * width * (4 + 4 + 2 + 2 + 2), 10.0 * T * width, VALU_F32))
        t = _time(lambda: _C.mixer_ops.gated_stream_step(stream, y[:, :width], y[:, width:], 0.5, hist, dw, norm, hout))
        rows.append(_row("gated_stream_step (+ history of %d layers mixed)" % depth, phase, t,
                         T * width * (4 + 4 + 2 + 2 + 2 + 4 * depth), (10.0 + 2 * depth) * T * width, VALU_F32))
        a = torch.randn(T, width, device=dev).to(bf)
        wgt = torch.zeros(width, device=dev)
        t2 = _time(lambda: _C.mixer_ops.stream_add_norm(stream, wgt, 1.0, 1e-6, hout, a, a, None))
        rows.append(_row("Lapilorn stream_add_norm (two addends)", phase, t2, T * width * (4 + 4 + 2 + 2 + 2), 6.0 * T * width, VALU_F32,
                         like="gated_stream_step"))
        # ---------------------------------------------------------------- feed-forward activation
        z = torch.randn(T, ff + width, device=dev).to(bf)
        act = torch.empty(T, ff, dtype=bf, device=dev)
        coef = torch.tensor([1.0, 0.3, 0.1, 0.0], device=dev)
        t = _time(lambda: _C.mixer_ops.poly_norm(act, z[:, :ff], coef, 1e-6))
        rows.append(_row("poly_norm", phase, t, T * ff * 2 * 2, 14.0 * T * ff, VALU_F32))
        gu = torch.randn(T, 2 * ff, device=dev).to(bf)
        t2 = _time(lambda: _C.mixer_ops.clamped_glu(act, gu, 1.702, 7.0, 1.0))
        rows.append(_row("Lapilorn clamped_glu", phase, t2, T * ff * 3 * 2, 8.0 * T * ff, VALU_F32, like="poly_norm"))
    return rows


@torch.inference_mode()
def kernel_table_bogetar(width: int = 2048, heads: int = 16, kv_heads: int = 4, prefill_rows: int = 4096,
                         decode_seqs: int = 64, decode_ctx: int = 2047, span: int = 1024, groups: int = 8, taps: int = 4,
                         experts: int = 32, top: int = 2, ff: int = 1408) -> List[dict]:
    """The kernels of the Bogetar layers beside their like: attention with sigmoid weights beside the same kernel with
    a softmax (as Lapilorn runs it, same window); the rotation kernel with the per-head norm beside the plain one; the
    delta rule with one decay per head beside Nepevik's with one per key channel; the grouped norm with its add beside
    the fused add + RMS norm; the convolution added to a sublayer's input beside the short convolution with silu; the
    softmax router beside the sigmoid router; experts with a gated hidden layer beside experts with relu^2."""
    from .. import _C
    dev, bf = torch.device("cuda"), torch.bfloat16
    d = width // heads
    page = 16
    rows: List[dict] = []
    scale = d ** -0.5
    for phase, seqs in (("prefill", [(0, prefill_rows // 2, 0, None), (0, prefill_rows // 2, 1, None)]),
                        ("decode", [(decode_ctx, 1, i, None) for i in range(decode_seqs)])):
        total_pages, laid = 0, []
        for ctx, n, slot, _ in seqs:
            pages = -(-(ctx + n) // page)
            laid.append((ctx, n, slot, list(range(total_pages, total_pages + pages))))
            total_pages += pages
        batch = _ragged(laid, dev)
        T, B = sum(s[1] for s in laid), len(laid)
        pairs = keys = 0
        for c, n, _, _ in laid:
            pairs += sum(min(i + 1, span) for i in range(c, c + n))
            keys += c + n - max(0, (c if n == 1 else 0) - span + 1)
        # ---------------------------------------------------------------- attention
        kc = torch.randn(total_pages, page, kv_heads * d, device=dev).to(bf)
        vc = torch.randn(total_pages, page, kv_heads * d, device=dev).to(bf)
        q = torch.randn(T, heads * d, device=dev)
        gate = torch.randn(T, heads * d, device=dev).to(bf)
        out = torch.empty(T, heads * d, dtype=bf, device=dev)
        bias = torch.full((heads,), -3.0, device=dev)
        abytes = keys * kv_heads * d * 2 * 2 + T * heads * d * (4 + 2 + 2)
        for name, kw, like in (("sigmoid attention (window %d, bias, gate)" % span, dict(score_bias=bias), ""),
                               ("capped_attention with a softmax, same window and gate", {}, "sigmoid attention")):
            t = _time(lambda: _C.mixer_ops.capped_attention(out, q, kc, vc, gate, batch, heads, kv_heads, d, d, scale, 0.0, span, **kw))
            rows.append(_row(name, phase, t, abytes, 4.0 * pairs * heads * d, VALU_F32, like=like))
        # ---------------------------------------------------------------- rotation and cache writes
        pos = torch.cat([torch.arange(c, c + n) for c, n, _, _ in laid]).to(dev)
        slots = torch.cat([torch.tensor([tb[p // page] * page + p % page for p in range(c, c + n)])
                           for c, n, _, tb in laid]).to(dev)
        proj = torch.randn(T, (heads + 2 * kv_heads) * d, device=dev).to(bf)
        inv = torch.rand(d // 4, device=dev)
        q32 = torch.empty(T, heads * d, device=dev)
        wq = torch.ones(d, device=dev)
        rbytes = T * ((heads + 2 * kv_heads) * d * 2 + heads * d * 4 + 2 * kv_heads * d * 2)
        for name, norm, like in (("rope_cache behind a per-head norm", (wq, wq, 1e-6), ""), ("rope_cache", (), "rope_cache + norm")):
            t = _time(lambda: _C.mixer_ops.rope_cache(q32, proj[:, :heads * d], proj[:, heads * d:(heads + kv_heads) * d],
                                                      proj[:, (heads + kv_heads) * d:], pos, inv, heads, kv_heads, d, d, kc,
                                                      vc, slots, True, *norm))
            rows.append(_row(name, phase, t, rbytes, (10.0 if norm else 6.0) * T * heads * d, VALU_F32, like=like))
        # ---------------------------------------------------------------- delta rules
        lbatch = _ragged([(c, n, i, []) for i, (c, n, _, _) in enumerate(laid)], dev)
        G = heads // 2
        c_ = 2 * G * d + heads * d
        dproj = torch.randn(T, c_ + 2 * heads, device=dev).to(bf)
        ctaps = torch.randn(c_, taps, device=dev) * 0.3
        cstate = torch.zeros(max(B, 2), taps - 1, c_, device=dev)
        rstate = torch.zeros(max(B, 2), heads, d, d, device=dev)
        qkv = torch.empty(T, c_, device=dev)
        o = torch.empty(T, heads * d, device=dev)
        zero_h, zero_hd = torch.zeros(heads, device=dev), torch.zeros(heads * d, device=dev)
        dpre = torch.randn(T, heads * d, device=dev).to(bf)
        t = _time(lambda: _C.mixer_ops.short_conv(qkv, dproj[:, :c_], ctaps, cstate, lbatch))
        rows.append(_row("short_conv + state advance (q | k | v, silu)", phase, t, T * c_ * (2 + 4), 2.0 * taps * T * c_, VALU_F32))
        dflops = T * heads * 6.0 * d * d
        dbytes = T * (c_ * 4 + heads * d * 4) + 2 * B * heads * d * d * 4
        t = _time(lambda: _C.mixer_ops.gated_delta(o, qkv, dproj[:, c_:c_ + heads], dproj[:, c_ + heads:], zero_h, zero_h, rstate,
                                                   lbatch, heads, G, d, d))
        rows.append(_row("gated_delta (one decay per head; prologue + recurrence)", phase, t, dbytes, dflops, VALU_F32))
        t = _time(lambda: _C.mixer_ops.channel_delta(o, qkv, dproj[:, c_:c_ + heads], dpre, zero_hd, zero_h, rstate, lbatch, heads,
                                                     G, d, d))
        rows.append(_row("Nepevik channel_delta (a decay per key channel), same sizes", phase, t, dbytes + T * heads * d * 2, dflops,
                         VALU_F32, like="gated_delta"))
        # ---------------------------------------------------------------- gated linear attention at this design's sizes
        rh, dk = heads // 4, d // 2
        gproj = torch.randn(T, rh * (2 * dk + d), device=dev).to(bf)
        zpre = torch.randn(T, rh * dk, device=dev).to(bf)
        zbias = torch.full((rh * dk,), 2.0, device=dev)
        gstate = torch.zeros(max(B, 2), rh, dk, d, device=dev)
        go = torch.empty(T, rh * d, device=dev)
        t = _time(lambda: _C.mixer_ops.gla(go, gproj[:, :rh * dk], gproj[:, rh * dk:2 * rh * dk], gproj[:, 2 * rh * dk:], zpre, zbias,
                                           16.0, dk ** -0.5, gstate, lbatch, rh, dk, d))
        rows.append(_row("gla (%d heads beside the attention)" % rh, phase, t,
                         T * rh * ((3 * dk + d) * 2 + d * 4) + 2 * B * rh * dk * d * 4,
                         T * rh * (2.0 * 32 * dk + 2.0 * 32 * d + 4.0 * dk * d), VALU_F32))
        # ---------------------------------------------------------------- norms and the convolution on a sublayer's input
        stream = torch.randn(T, width, device=dev)
        y = torch.randn(T, 2 * width, device=dev).to(bf)
        y32 = torch.randn(T, width, device=dev)
        wn = torch.ones(width, device=dev)
        h32 = torch.empty(T, width, device=dev)
        t = _time(lambda: _C.mixer_ops.group_norm_add(stream, groups, 1e-6, y[:, :width], wn, wn, None, 1.0, 1.0, wn, h32))
        rows.append(_row("group_norm_add (one addend, %d groups, fp32 norm out)" % groups, phase, t, T * width * (4 + 4 + 2 + 4),
                         12.0 * T * width, VALU_F32))
        t = _time(lambda: _C.mixer_ops.group_norm_add(stream, groups, 1e-6, y[:, :width], wn, wn, y[:, width:], 0.8, 0.5, wn, h32))
        rows.append(_row("group_norm_add (two addends)", phase, t, T * width * (4 + 4 + 2 + 2 + 4), 14.0 * T * width, VALU_F32))
        t = _time(lambda: _C.mixer_ops.group_norm_add(stream, groups, 1e-6, y32, wn, wn, None, 1.0, 1.0, wn, h32))
        rows.append(_row("group_norm_add (fp32 addend: the experts' sum)", phase, t, T * width * (4 + 4 + 4 + 4), 12.0 * T * width,
                         VALU_F32))
        hout = torch.empty(T, width, dtype=bf, device=dev)
        t2 = _time(lambda: _C.mixer_ops.stream_add_norm(stream, wn, 1.0, 1e-6, hout, y[:, :width], y[:, width:], None))
        rows.append(_row("Lapilorn stream_add_norm (two addends)", phase, t2, T * width * (4 + 4 + 2 + 2 + 2), 6.0 * T * width, VALU_F32,
                         like="group_norm_add"))
        wtaps = torch.randn(width, taps, device=dev) * 0.3
        wstate = torch.zeros(max(B, 2), taps - 1, width, device=dev)
        t = _time(lambda: _C.mixer_ops.causal_conv(hout, h32, wtaps, wstate, lbatch))
        rows.append(_row("causal_conv added to its input + state advance (fp32 in)", phase, t, T * width * (4 + 2), 2.0 * taps * T * width,
                         VALU_F32, like="short_conv"))
        # ---------------------------------------------------------------- router and experts
        logits = torch.randn(T, experts, device=dev)
        t = _time(lambda: _C.mixer_ops.group_router(logits, None, top, 4, 2, 1.0, True, True, False))
        rows.append(_row("group_router (softmax, best-of-group, weights as they are)", phase, t, T * experts * 4 + T * top * 8,
                         8.0 * T * experts, VALU_F32))
        t2 = _time(lambda: _C.mixer_ops.group_router(logits, None, top, 4, 2, 1.0))
        rows.append(_row("Lapilorn group_router (sigmoid)", phase, t2, T * experts * 4 + T * top * 8, 8.0 * T * experts, VALU_F32,
                         like="group_router"))
        chosen, weights = _C.mixer_ops.group_router(logits, None, top, 4, 2, 1.0, True, True, False)
        order, start = _C.mixer_ops.group_pairs(chosen, experts)
        x = torch.randn(T, width, device=dev).to(bf)
        up_glu = (torch.randn(experts, 32 * (-(-ff // 16)), width, device=dev) * 0.02).to(bf)
        down = (torch.randn(experts, width, ff, device=dev) * 0.02).to(bf)
        eo = torch.zeros(T, width, device=dev)
        active = min(experts, T * top)
        ebytes = active * 3 * ff * width * 2 + T * width * (2 + 4) + T * top * ff * 2 * 2
        t = _time(lambda: _C.mixer_ops.expert_ffn(eo, x, up_glu, down, order, start, top, 1.0, pair_weight=weights,
                                                  glu=(1.702, 7.0, 1.0)))
        rows.append(_row("expert_ffn (gated hidden layer with limits)", phase, t, ebytes, 6.0 * T * top * ff * width, MFMA_BF16))
        ff2 = 3 * ff // 2                                  # relu^2 experts of the same weights' size: up + down of 1.5 ff
        up_r = (torch.randn(experts, ff2, width, device=dev) * 0.02).to(bf)
        down_r = (torch.randn(experts, width, ff2, device=dev) * 0.02).to(bf)
        t2 = _time(lambda: _C.mixer_ops.expert_ffn(eo, x, up_r, down_r, order, start, top, 1.0, activation=_C.mixer_ops.ACT_RELU2,
                                                   pair_weight=weights))
        rows.append(_row("Lapilorn expert_ffn (relu^2), same weights' size", phase, t2,
                         active * 2 * ff2 * width * 2 + T * width * (2 + 4) + T * top * ff2 * 2 * 2, 4.0 * T * top * ff2 * width,
                         MFMA_BF16, like="expert_ffn"))
    return rows


def run(sizes=("2k",), with_kernels: bool = True, family: str = "nepevik") -> dict:
    result = {"family": family, "engine": {}, "kernels": {}}
    for size in sizes:
        pair = {}
        for name in (family, "llama"):
            pair[name] = {k: round(v, 2) for k, v in engine_throughput(f"{name}-{size}").items()}
        result["engine"][size] = pair
    if with_kernels:
        table = {"nepevik": kernel_table, "lapilorn": kernel_table_lapilorn, "lalasun": kernel_table_lalasun,
                 "bogetar": kernel_table_bogetar}[family]
        result["kernels"]["2k"] = table()
    return result

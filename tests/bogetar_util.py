"""Small random Bogetar models on disk.  The engine harness (``Replayer``, ``make_engine``, ``write_model``,
``row_error``) is the one of ``nepevik_util``: it only speaks to the engine."""
from typing import Dict, List, Optional

import torch

from nepevik_util import Replayer, make_engine, row_error, write_model  # noqa: F401  (re-exported)


def delta(heads=3, kv_heads=3, dim=12, vdim=8, conv=4):
    return {"type": "delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}}


def parallel(heads=4, kv_heads=2, dim=16, vdim=24, window=9, scale=0.3, rot_dims=8, base=100.0, r_heads=3, r_dim=10,
             r_vdim=12, tau=4.0, left_scale=0.7, right_scale=1.2):
    return {"type": "parallel",
            "mixer": {"left": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale,
                               "mask": {"size": window}, "rot": {"base": base, "dims": rot_dims}},
                      "right": {"heads": r_heads, "dim": r_dim, "vdim": r_vdim, "tau": tau},
                      "left_scale": left_scale, "right_scale": right_scale}}


def moe(experts=6, top=2, ff=20, groups=3, keep=2, limit=1.0):
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit},
            "router": {"experts": experts, "top": top, "groups": {"count": groups, "keep": keep}}}


def config(layers: List[dict], mlps: List[Optional[dict]], vocab=97, width=48, eps=1e-5, groups=4, taps=3) -> dict:
    out = []
    for layer, mlp in zip(layers, mlps):
        entry = dict(layer)
        entry["mlp"] = mlp
        out.append(entry)
    return {"architecture": "Bogetar", "canon": {"taps": taps}, "layers": out, "norm": {"eps": eps, "groups": groups},
            "vocab": vocab, "width": width}


def random_weights(cfg: dict, seed: int, decay_rank=5) -> Dict[str, torch.Tensor]:
    """bf16 weights under the checkpoint's names; magnitudes chosen so that every mechanism matters: norm weights and
    layer scales spread around their means, convolution taps of a size that counts, score biases that leave most
    keys a small weight, decays from nearly none to strong, limits that bite, routers whose groups disagree."""
    g = torch.Generator().manual_seed(seed)
    width, vocab = cfg["width"], cfg["vocab"]
    taps = cfg["canon"]["taps"]

    def rnd(*shape, scale=1.0, mean=0.0):
        return (torch.randn(tuple(shape), generator=g) * scale + mean).to(torch.bfloat16)

    def lin(out, inp, gain=1.0):
        return rnd(out, inp, scale=gain / inp ** 0.5)

    sd = {"embed": rnd(vocab, width), "final.norm": rnd(width, scale=0.2, mean=1.0)}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        subs = ("1", "2") if layer.get("mlp") is not None else ("1",)
        for s in subs:
            sd[p + "norm" + s] = rnd(width, scale=0.2, mean=1.0)
            sd[p + "norm" + s + "b"] = rnd(width, scale=0.2, mean=1.0)
            sd[p + "ls" + s] = rnd(width, scale=0.15, mean=0.6)
            sd[p + "canon" + s] = rnd(width, taps, scale=0.4)
        if layer["type"] == "delta":
            h, kv, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            for name, size in (("q", kv * d), ("k", kv * d), ("v", h * dv)):
                sd[p + f"mix.{name}"] = lin(size, width, 2.0)
                sd[p + f"mix.{name}.conv"] = rnd(size, m["conv"], scale=0.6)
            sd[p + "mix.b"], sd[p + "mix.a"] = lin(h, width, 2.0), lin(h, width, 2.0)
            sd[p + "mix.A_log"], sd[p + "mix.dt_bias"] = rnd(h, scale=0.7), rnd(h, scale=1.0)
            sd[p + "mix.norm"] = rnd(dv, scale=0.3, mean=1.0)
            sd[p + "mix.g"], sd[p + "mix.o"] = lin(h * dv, width, 2.0), lin(width, h * dv)
        else:
            left, right = m["left"], m["right"]
            h, kv, d, dv = left["heads"], left["kv_heads"], left["dim"], left["vdim"]
            q = p + "mix.left."
            sd[q + "q"], sd[q + "k"], sd[q + "v"] = lin(h * d, width, 3.0), lin(kv * d, width, 3.0), lin(kv * dv, width)
            sd[q + "q.norm"], sd[q + "k.norm"] = rnd(d, scale=0.3, mean=1.2), rnd(d, scale=0.3, mean=1.2)
            sd[q + "pb"] = rnd(h, scale=0.7, mean=-1.5)
            sd[q + "g"], sd[q + "o"] = lin(h * dv, width, 2.0), lin(width, h * dv)
            rh, rd, rdv = right["heads"], right["dim"], right["vdim"]
            r = p + "mix.right."
            sd[r + "q"], sd[r + "k"] = lin(rh * rd, width, 2.0), lin(rh * rd, width, 2.0)
            sd[r + "v"], sd[r + "g"] = lin(rh * rdv, width, 1.5), lin(rh * rdv, width, 2.0)
            sd[r + "a1"], sd[r + "a2"] = lin(decay_rank, width, 2.0), lin(rh * rd, decay_rank, 3.0)
            sd[r + "a2.b"] = rnd(rh * rd, scale=1.5, mean=1.0)
            sd[r + "norm"] = rnd(rdv, scale=0.3, mean=1.0)
            sd[r + "o"] = lin(width, rh * rdv)
        mlp = layer.get("mlp")
        if mlp is not None:
            ff = mlp["expert"]["ff"]
            sd[p + "mlp.router"] = lin(mlp["router"]["experts"], width, 3.0)
            for e in range(mlp["router"]["experts"]):
                sd[p + f"mlp.e{e}.gate"], sd[p + f"mlp.e{e}.up"] = lin(ff, width, 2.0), lin(ff, width, 2.0)
                sd[p + f"mlp.e{e}.down"] = lin(width, ff, 1.5)
    return sd


def share_within(got: torch.Tensor, want: torch.Tensor, tol: float) -> float:
    """The share of positions whose logits lie within ``tol`` (errors as ``row_error`` measures them, per position).
    In bf16 a router's close call may fall the other way and move a position (and, through the recurrent states, a
    few after it) by much more than rounding does: a bf16 comparison asks for most positions, not for every one."""
    d = got.double() - want.double()
    d = d - d.mean(-1, keepdim=True)
    scale = (want.double() - want.double().mean(-1, keepdim=True)).pow(2).mean().sqrt()
    return float(((d.pow(2).mean(-1).sqrt() / scale) < tol).double().mean())

"""Small random Lalasun models on disk.  The engine harness (``Replayer``, ``make_engine``, ``write_model``,
``row_error``) is the one of ``nepevik_util``: it only speaks to the engine."""
from typing import Dict, List, Optional

import torch

from nepevik_util import Replayer, make_engine, row_error, write_model  # noqa: F401  (re-exported)


def latent(heads=3, dim=8, rot_dim=4, vdim=12, kv_rank=20, window=9, scale=0.35, base=40.0):
    return {"type": "latent_attention",
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale,
                      "mask": {"size": window}, "rot": {"base": base, "dims": rot_dim}}}


def attention(heads=4, kv_heads=2, dim=16, vdim=8, chunk=11, scale=0.3, rot_dims=8, base=100.0):
    return {"type": "attention",
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale,
                      "mask": {"size": chunk}, "rot": {"base": base, "dims": rot_dims}}}


def gla(heads=2, dim=12, vdim=20, tau=4.0):
    return {"type": "gla", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau}}


def dense(ff=40):
    return {"kind": "dense", "ff": ff}


def config(layers: List[dict], mlps: List[Optional[dict]], vocab=97, width=48, eps=1e-5, mult=0.8) -> dict:
    out = []
    for layer, mlp in zip(layers, mlps):
        entry = dict(layer)
        entry["mlp"] = mlp
        out.append(entry)
    return {"architecture": "Lalasun", "layers": out, "norm": {"eps": eps}, "residual_mult": mult, "vocab": vocab,
            "width": width}


def random_weights(cfg: dict, seed: int, decay_rank=5) -> Dict[str, torch.Tensor]:
    """bf16 weights under the checkpoint's names; magnitudes chosen so that every mechanism matters: norms whose
    tanh bends, gates spread around one half, decays from nearly none to strong, activation numbers that all count,
    depth weights that reach back to the embedding."""
    g = torch.Generator().manual_seed(seed)
    width, vocab = cfg["width"], cfg["vocab"]

    def rnd(*shape, scale=1.0):
        return (torch.randn(tuple(shape), generator=g) * scale).to(torch.bfloat16)

    def lin(out, inp, gain=1.0):
        return rnd(out, inp, scale=gain / inp ** 0.5)

    def norm(name):
        sd[name] = rnd(width, scale=0.2) + 1.0
        sd[name + ".b"] = rnd(width, scale=0.1)
        sd[name + ".alpha"] = (0.4 + 0.4 * torch.rand((), generator=g)).to(torch.bfloat16)

    sd = {"embed": rnd(vocab, width), "head": lin(vocab, width)}
    norm("final.norm")
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        norm(p + "norm1")
        h, d = m["heads"], m["dim"]
        dv = m.get("vdim", d)
        if layer["type"] == "latent_attention":
            dr, rank = m["rot_dim"], m["kv_rank"]
            sd[p + "mix.q"] = lin(h * (d + dr), width, 3.0)
            sd[p + "mix.dkv"] = lin(rank + dr, width, 2.0)
            sd[p + "mix.dkv.norm"] = rnd(rank, scale=0.3) + 1.0
            sd[p + "mix.uk"], sd[p + "mix.uv"] = lin(h * d, rank, 1.5), lin(h * dv, rank)
            sd[p + "mix.g"] = lin(h * dv, width, 2.0)
        elif layer["type"] == "attention":
            kv = m.get("kv_heads", h)
            for name, size, gain in (("q", h * d, 3.0), ("k", kv * d, 3.0), ("v", kv * dv, 1.0)):
                sd[p + f"mix.{name}"] = lin(size, width, gain)
                sd[p + f"mix.{name}.b"] = rnd(size, scale=0.3)
            sd[p + "mix.o.b"] = rnd(width, scale=0.2)
        else:
            sd[p + "mix.q"], sd[p + "mix.k"] = lin(h * d, width, 2.0), lin(h * d, width, 2.0)
            sd[p + "mix.v"], sd[p + "mix.g"] = lin(h * dv, width, 1.5), lin(h * dv, width, 2.0)
            sd[p + "mix.a1"], sd[p + "mix.a2"] = lin(decay_rank, width, 2.0), lin(h * d, decay_rank, 3.0)
            sd[p + "mix.a2.b"] = rnd(h * d, scale=1.5) + 1.0
            sd[p + "mix.norm"] = rnd(dv, scale=0.3) + 1.0
        sd[p + "mix.o"] = lin(width, h * dv)
        sd[p + "rg1"], sd[p + "rg1.b"] = lin(width, width, 2.0), rnd(width, scale=0.5)
        if layer.get("mlp") is not None:
            norm(p + "norm2")
            ff = layer["mlp"]["ff"]
            sd[p + "mlp.up"], sd[p + "mlp.down"] = lin(ff, width, 2.0), lin(width, ff)
            sd[p + "mlp.act"] = torch.tensor([0.9, 0.4, -0.3, 0.1]).to(torch.bfloat16)
            sd[p + "rg2"], sd[p + "rg2.b"] = lin(width, width, 2.0), rnd(width, scale=0.5)
        w = 0.3 * torch.randn(i + 2, generator=g)
        w[-1] += 1.0
        sd[p + "dwa"] = w.to(torch.bfloat16)
    return sd

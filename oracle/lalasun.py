"""Plain, slow CPU statement of the Lalasun decoder -- TEST INFRASTRUCTURE ONLY.

One function per mechanism, token-by-token loops, no cache, no batching; nothing here is shared with the
engine's model code.  ``logits`` runs a whole token sequence and returns the logits of every position (and,
on request, the stream after every layer).

Notation.  x: the stream a layer receives [n, width]; r: config ``residual_mult``.
    h1 = T1(x);  y = x + r * mixer(h1) * sigmoid(G1 h1 + g1)
    h2 = T2(y);  X = y + r * ff(h2)    * sigmoid(G2 h2 + g2)
    T(u) = tanh(a * u) * w + b   (a: one number per norm)
With X_0 the embedding rows and X_(i+1) layer i's X, the next layer (or the output) receives
    sum_{j <= i+1} D_i[j] X_j        (D_i: the layer's i + 2 depth weights)
Weights are [out, in] and applied as W u.  The logits come from a matrix of their own.
"""
from typing import Dict, List

import torch


def tanh_norm(u: torch.Tensor, a: torch.Tensor, w: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    return torch.tanh(a * u) * w + b


def rms_unit(u: torch.Tensor, eps: float) -> torch.Tensor:
    return u / torch.sqrt(u.pow(2).mean(-1, keepdim=True) + eps)


def poly_norm(z: torch.Tensor, coef: torch.Tensor, eps: float) -> torch.Tensor:
    """coef = (a, b, c, e): a U(z) + b U(z^2) + c U(z^3) + e, U = division by the root mean square over the row."""
    return coef[0] * rms_unit(z, eps) + coef[1] * rms_unit(z * z, eps) + coef[2] * rms_unit(z * z * z, eps) + coef[3]


def rotary_frequencies(rot: dict) -> List[float]:
    return [rot["base"] ** (-2.0 * i / rot["dims"]) for i in range(rot["dims"] // 2)]


def _angle(position: int, f: float, dtype) -> torch.Tensor:
    # fp32 position times fp32 frequency, as the design computes it
    return (torch.tensor(float(position), dtype=torch.float32) * torch.tensor(f, dtype=torch.float32)).to(
        torch.float64)


def rotate_neighbours(y: torch.Tensor, position: int, freqs: List[float]) -> torch.Tensor:
    """y [heads, size]: pairs (2i, 2i + 1) of the first 2 * len(freqs) coordinates turn by position * f_i."""
    out = y.clone()
    for i, f in enumerate(freqs):
        a = _angle(position, f, y.dtype)
        c, s = torch.cos(a).to(y.dtype), torch.sin(a).to(y.dtype)
        u, v = y[:, 2 * i], y[:, 2 * i + 1]
        out[:, 2 * i] = u * c - v * s
        out[:, 2 * i + 1] = v * c + u * s
    return out


def rotate_halves(y: torch.Tensor, position: int, freqs: List[float]) -> torch.Tensor:
    """y [heads, size]: pairs (i, i + len(freqs)) of the first 2 * len(freqs) coordinates turn by position * f_i."""
    out = y.clone()
    n = len(freqs)
    for i, f in enumerate(freqs):
        a = _angle(position, f, y.dtype)
        c, s = torch.cos(a).to(y.dtype), torch.sin(a).to(y.dtype)
        u, v = y[:, i], y[:, i + n]
        out[:, i] = u * c - v * s
        out[:, i + n] = v * c + u * s
    return out


def masked_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, window: int = 0, chunk: int = 0,
                     sink: bool = False, first_position: int = 0) -> torch.Tensor:
    """q [n, H, d] at positions first_position ..; k [m, G, d], v [m, G, dv] from position 0.  -> [n, H, dv].
    Query head a reads key/value head a // (H // G).  Position i sees j <= i, with ``window`` only i - j < window,
    with ``chunk`` only j // chunk == i // chunk.  ``sink``: the weights are exp(s_j) / (1 + sum exp(s_j))."""
    n, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(n, H, v.shape[2], dtype=q.dtype)
    for t in range(n):
        pos = first_position + t
        lo = max(0, pos - window + 1) if window else (pos // chunk) * chunk if chunk else 0
        for a in range(H):
            g = a // (H // G)
            s = (k[lo:pos + 1, g] @ q[t, a]) * scale
            if sink:
                e = torch.exp(s)
                p = e / (1.0 + e.sum())
            else:
                p = torch.softmax(s, 0)
            out[t, a] = p @ v[lo:pos + 1, g]
    return out


def latent_attention_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict, eps: float) -> torch.Tensor:
    """Keys and values of all heads come from one small latent per token; one rotated key part is shared by the
    heads; sliding window; sigmoid gate on the heads' output."""
    n = h.shape[0]
    H, d, dr, dv, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    freqs = rotary_frequencies(m["rot"])
    assert m["rot"]["dims"] == dr
    q = (h @ w["q"].T).view(n, H, d + dr)
    down = h @ w["dkv"].T
    latent = rms_unit(down[:, :rank], eps) * w["dkv.norm"]
    k_rot = torch.stack([rotate_neighbours(down[t:t + 1, rank:], t, freqs)[0] for t in range(n)])
    q_rot = torch.stack([rotate_neighbours(q[t, :, d:], t, freqs) for t in range(n)])
    k_plain = (latent @ w["uk"].T).view(n, H, d)
    v = (latent @ w["uv"].T).view(n, H, dv)
    # a head's key is its own plain part next to the part that all heads share
    k_full = torch.cat([k_plain, k_rot.unsqueeze(1).expand(n, H, dr)], -1)
    q_full = torch.cat([q[:, :, :d], q_rot], -1)
    out = masked_attention(q_full, k_full, v, m["scale"], window=m["mask"]["size"])
    gate = torch.sigmoid(h @ w["g"].T)
    return (out.reshape(n, H * dv) * gate) @ w["o"].T


def chunked_sink_attention_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict) -> torch.Tensor:
    """Grouped query heads with biased projections; a position sees the earlier positions of its own chunk of
    ``mask.size``; the softmax has one more term in its denominator (score 0, no value)."""
    n = h.shape[0]
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    G = m.get("kv_heads", H)
    freqs = rotary_frequencies(m["rot"])
    q = (h @ w["q"].T + w["q.b"]).view(n, H, d)
    k = (h @ w["k"].T + w["k.b"]).view(n, G, d)
    v = (h @ w["v"].T + w["v.b"]).view(n, G, dv)
    q = torch.stack([rotate_halves(q[t], t, freqs) for t in range(n)])
    k = torch.stack([rotate_halves(k[t], t, freqs) for t in range(n)])
    out = masked_attention(q, k, v, m["scale"], chunk=m["mask"]["size"], sink=True)
    return out.reshape(n, H * dv) @ w["o"].T + w["o.b"]


def decayed_state_scan(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, decay: torch.Tensor, state=None):
    """q, k, decay [n, H, d], v [n, H, dv]:  S <- diag(decay_t) S + k_t v_t^T;  o_t = S^T q_t.  -> (o [n, H, dv], S)."""
    n, H, d = q.shape
    S = torch.zeros(H, d, v.shape[2], dtype=q.dtype) if state is None else state.clone()
    o = torch.zeros(n, H, v.shape[2], dtype=q.dtype)
    for t in range(n):
        S = decay[t].unsqueeze(-1) * S + k[t].unsqueeze(-1) * v[t].unsqueeze(-2)
        o[t] = torch.einsum("hdv,hd->hv", S, q[t])
    return o, S


def channel_decay(z: torch.Tensor, tau: float) -> torch.Tensor:
    """sigmoid(z)^(1 / tau), through the logarithm."""
    return torch.exp(torch.nn.functional.logsigmoid(z) / tau)


def gla_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict, eps: float) -> torch.Tensor:
    """Gated linear attention: a decay per head and key channel from a low-rank projection of the input."""
    n = h.shape[0]
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    q = (h @ w["q"].T).view(n, H, d) * d ** -0.5
    k = (h @ w["k"].T).view(n, H, d)
    v = (h @ w["v"].T).view(n, H, dv)
    decay = channel_decay((h @ w["a1"].T) @ w["a2"].T + w["a2.b"], m["tau"]).view(n, H, d)
    o, _ = decayed_state_scan(q, k, v, decay)
    o = rms_unit(o, eps) * w["norm"]
    gate = h @ w["g"].T
    return (o.reshape(n, H * dv) * (gate * torch.sigmoid(gate))) @ w["o"].T


def feed_forward(h: torch.Tensor, w: Dict[str, torch.Tensor], mlp: dict, eps: float) -> torch.Tensor:
    if mlp["kind"] != "dense":
        raise ValueError(mlp["kind"])
    return poly_norm(h @ w["up"].T, w["act"], eps) @ w["down"].T


def logits(cfg: dict, weights: Dict[str, torch.Tensor], tokens: List[int], dtype=torch.float64,
           keep_streams: bool = False):
    """-> logits [n, vocab] (and the stream handed on after every layer)."""
    W = {k: (v.to(dtype) if v.dtype.is_floating_point else v) for k, v in weights.items()}
    eps, r = cfg["norm"]["eps"], cfg["residual_mult"]

    def sub(prefix):
        return {k[len(prefix):]: v for k, v in W.items() if k.startswith(prefix)}

    def norm(u, name):
        return tanh_norm(u, W[name + ".alpha"], W[name], W[name + ".b"])

    x = W["embed"][torch.tensor(tokens)]
    outputs, streams = [x], []
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        h = norm(x, p + "norm1")
        if layer["type"] == "latent_attention":
            a = latent_attention_mixer(h, sub(p + "mix."), m, eps)
        elif layer["type"] == "attention":
            a = chunked_sink_attention_mixer(h, sub(p + "mix."), m)
        elif layer["type"] == "gla":
            a = gla_mixer(h, sub(p + "mix."), m, eps)
        else:
            raise ValueError(layer["type"])
        x = x + r * a * torch.sigmoid(h @ W[p + "rg1"].T + W[p + "rg1.b"])
        if layer.get("mlp") is not None:
            h = norm(x, p + "norm2")
            x = x + r * feed_forward(h, sub(p + "mlp."), layer["mlp"], eps) * torch.sigmoid(
                h @ W[p + "rg2"].T + W[p + "rg2.b"])
        outputs.append(x)
        x = sum(W[p + "dwa"][j] * outputs[j] for j in range(i + 2))
        streams.append(x)
    out = norm(x, "final.norm") @ W["head"].T
    return (out, streams) if keep_streams else out

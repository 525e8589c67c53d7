"""Plain, slow CPU statement of the Bogetar decoder -- TEST INFRASTRUCTURE ONLY.

One function per mechanism, token-by-token loops, no cache, no batching; nothing here is shared with the
engine's model code.  ``logits`` runs a whole token sequence and returns the logits of every position (and,
on request, the stream after every layer).

Notation.  x: the stream a layer receives [n, width].  N(u; w): u cut into ``norm.groups`` equal runs, each run
divided by its own root mean square (eps inside the root), the whole times w.  C(u; c): u_t + sum_j c[:, j] *
u_(t - taps + 1 + j), a causal convolution per channel added to its own input (rows before the sequence count 0).
    a = C(N(x; norm1); canon1);   x = x + ls1 * N(mixer(a); norm1b)
    b = C(N(x; norm2); canon2);   x = x + ls2 * N(ff(b); norm2b)
Weights are [out, in] and applied as W u.  The logits reuse the embedding table.
"""
import math
from typing import Dict, List, Optional

import torch


def group_norm(u: torch.Tensor, w: torch.Tensor, groups: int, eps: float) -> torch.Tensor:
    """u [..., width]: every run of width / groups coordinates over its own root mean square, then times w."""
    parts = u.unflatten(-1, (groups, u.shape[-1] // groups))
    parts = parts / torch.sqrt(parts.pow(2).mean(-1, keepdim=True) + eps)
    return parts.flatten(-2) * w


def causal_conv(u: torch.Tensor, taps: torch.Tensor) -> torch.Tensor:
    """u [n, channels], taps [channels, T] (last column: the current token) -> sum_j taps[:, j] u_(t - T + 1 + j)."""
    n, T = u.shape[0], taps.shape[1]
    out = torch.zeros_like(u)
    for t in range(n):
        for j in range(T):
            src = t - T + 1 + j
            if src >= 0:
                out[t] += taps[:, j] * u[src]
    return out


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def unit(z: torch.Tensor) -> torch.Tensor:
    """z [..., size] -> z / sqrt(sum z^2 + 1e-6)."""
    return z / torch.sqrt(z.pow(2).sum(-1, keepdim=True) + 1e-6)


def softplus(z: torch.Tensor) -> torch.Tensor:
    return torch.clamp(z, min=0) + torch.log1p(torch.exp(-z.abs()))


def rotary_frequencies(rot: dict) -> List[float]:
    return [rot["base"] ** (-2.0 * i / rot["dims"]) for i in range(rot["dims"] // 2)]


def rotate_halves(y: torch.Tensor, position: int, freqs: List[float]) -> torch.Tensor:
    """y [heads, size]: pairs (i, i + len(freqs)) of the first 2 * len(freqs) coordinates turn by position * f_i
    (fp32 position times fp32 frequency, as the design computes the angle)."""
    out = y.clone()
    n = len(freqs)
    for i, f in enumerate(freqs):
        a = (torch.tensor(float(position), dtype=torch.float32) * torch.tensor(f, dtype=torch.float32)).double()
        c, s = torch.cos(a).to(y.dtype), torch.sin(a).to(y.dtype)
        u, v = y[:, i], y[:, i + n]
        out[:, i] = u * c - v * s
        out[:, i + n] = v * c + u * s
    return out


def sigmoid_window_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, bias: torch.Tensor, scale: float,
                             window: int, first_position: int = 0) -> torch.Tensor:
    """q [n, H, d] at positions first_position ..; k [m, G, d], v [m, G, dv] from position 0; bias [H].
    Position i sees j with 0 <= i - j < window; a seen key weighs sigmoid(q . k * scale + bias[head]); the weights
    are not normalised.  Query head a reads key/value head a // (H // G).  -> [n, H, dv]."""
    n, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(n, H, v.shape[2], dtype=q.dtype)
    for t in range(n):
        pos = first_position + t
        lo = max(0, pos - window + 1)
        for a in range(H):
            g = a // (H // G)
            s = (k[lo:pos + 1, g] @ q[t, a]) * scale + bias[a]
            out[t, a] = torch.sigmoid(s) @ v[lo:pos + 1, g]
    return out


def gated_delta_scan(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, beta: torch.Tensor, decay: torch.Tensor,
                     state: Optional[torch.Tensor] = None):
    """q, k [n, H, d], v [n, H, dv], beta, decay [n, H]; state [H, d, dv] (None: zeros).
    S <- decay S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q.  -> (o [n, H, dv], state)."""
    n, H, d = q.shape
    S = torch.zeros(H, d, v.shape[2], dtype=q.dtype) if state is None else state.clone()
    out = torch.zeros(n, H, v.shape[2], dtype=q.dtype)
    for t in range(n):
        for a in range(H):
            S[a] = decay[t, a] * S[a]
            u = beta[t, a] * (v[t, a] - S[a].t() @ k[t, a])
            S[a] = S[a] + torch.outer(k[t, a], u)
            out[t, a] = S[a].t() @ q[t, a]
    return out, S


def channel_decay_scan(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, alpha: torch.Tensor,
                       state: Optional[torch.Tensor] = None):
    """q, k, alpha [n, H, d], v [n, H, dv].  S <- diag(alpha_t) S + k_t v_t^T;  o_t = S^T q_t."""
    n, H, d = q.shape
    S = torch.zeros(H, d, v.shape[2], dtype=q.dtype) if state is None else state.clone()
    out = torch.zeros(n, H, v.shape[2], dtype=q.dtype)
    for t in range(n):
        for a in range(H):
            S[a] = alpha[t, a].unsqueeze(1) * S[a] + torch.outer(k[t, a], v[t, a])
            out[t, a] = S[a].t() @ q[t, a]
    return out, S


def head_rms(o: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """o [n, H, dv]: every head over its own root mean square, times w [dv]."""
    return o / torch.sqrt(o.pow(2).mean(-1, keepdim=True) + eps) * w


def route(z: torch.Tensor, top: int, groups: int, keep: int):
    """z [experts]: router logits of one token -> (chosen expert ids, their weights).  Scores are the softmax over
    all experts; a group of neighbouring experts scores its largest score; only experts of the ``keep`` best groups
    can be chosen; the ``top`` largest scores among them are chosen and weigh their own score."""
    s = torch.softmax(z, -1)
    E = s.numel()
    size = E // groups
    group_score = s.view(groups, size).max(-1).values
    kept = torch.topk(group_score, keep).indices.tolist()
    allowed = torch.full((E,), -1.0, dtype=s.dtype)
    for g in kept:
        allowed[g * size:(g + 1) * size] = s[g * size:(g + 1) * size]
    chosen = torch.topk(allowed, top).indices
    return chosen, s[chosen]


def expert(h: torch.Tensor, gate: torch.Tensor, up: torch.Tensor, down: torch.Tensor, limit: float) -> torch.Tensor:
    g = torch.clamp(gate @ h, max=limit)
    u = torch.clamp(up @ h, -limit, limit)
    return down @ (g * torch.sigmoid(1.702 * g) * (u + 1.0))


# ------------------------------------------------------------------------------------------------ sublayers
def delta_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict, eps: float) -> torch.Tensor:
    n = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]

    def branch(name):
        z = h @ w[name].t()
        return silu(causal_conv(z, w[name + ".conv"]))
    q = unit(branch("q").view(n, G, d)) * d ** -0.5
    k = unit(branch("k").view(n, G, d))
    v = branch("v").view(n, H, dv)
    rep = H // G
    q, k = q.repeat_interleave(rep, 1), k.repeat_interleave(rep, 1)
    beta = torch.sigmoid(h @ w["b"].t())
    decay = torch.exp(-torch.exp(w["A_log"]) * softplus(h @ w["a"].t() + w["dt_bias"]))
    o, _ = gated_delta_scan(q, k, v, beta, decay)
    o = head_rms(o, w["norm"], eps) * silu(h @ w["g"].t()).view(n, H, dv)
    return o.reshape(n, H * dv) @ w["o"].t()


def left_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict, eps: float) -> torch.Tensor:
    n = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w["q"].t()).view(n, H, d)
    k = (h @ w["k"].t()).view(n, G, d)
    v = (h @ w["v"].t()).view(n, G, dv)
    q = q / torch.sqrt(q.pow(2).mean(-1, keepdim=True) + eps) * w["q.norm"]
    k = k / torch.sqrt(k.pow(2).mean(-1, keepdim=True) + eps) * w["k.norm"]
    freqs = rotary_frequencies(m["rot"])
    q = torch.stack([rotate_halves(q[t], t, freqs) for t in range(n)])
    k = torch.stack([rotate_halves(k[t], t, freqs) for t in range(n)])
    o = sigmoid_window_attention(q, k, v, w["pb"], m["scale"], m["mask"]["size"])
    o = o.reshape(n, H * dv) * torch.sigmoid(h @ w["g"].t())
    return o @ w["o"].t()


def right_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict, eps: float) -> torch.Tensor:
    n = h.shape[0]
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    q = (h @ w["q"].t()).view(n, H, d) * d ** -0.5
    k = (h @ w["k"].t()).view(n, H, d)
    v = (h @ w["v"].t()).view(n, H, dv)
    z = (h @ w["a1"].t()) @ w["a2"].t() + w["a2.b"]
    alpha = torch.sigmoid(z).pow(1.0 / m["tau"]).view(n, H, d)
    o, _ = channel_decay_scan(q, k, v, alpha)
    o = head_rms(o, w["norm"], eps).reshape(n, H * dv) * silu(h @ w["g"].t())
    return o @ w["o"].t()


def parallel_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict, eps: float) -> torch.Tensor:
    left = left_mixer(h, {k[5:]: v for k, v in w.items() if k.startswith("left.")}, m["left"], eps)
    right = right_mixer(h, {k[6:]: v for k, v in w.items() if k.startswith("right.")}, m["right"], eps)
    return m["left_scale"] * left + m["right_scale"] * right


def experts_ff(h: torch.Tensor, w: Dict[str, torch.Tensor], mlp: dict) -> torch.Tensor:
    r = mlp["router"]
    groups = r.get("groups") or {"count": 1, "keep": 1}
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        z = w["router"].float().double() @ h[t]
        chosen, weights = route(z, r["top"], groups["count"], groups["keep"])
        for e, s in zip(chosen.tolist(), weights):
            out[t] += s * expert(h[t], w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"], mlp["expert"]["limit"])
    return out


# ---------------------------------------------------------------------------------------------------- model
def logits(cfg: dict, weights: Dict[str, torch.Tensor], tokens: List[int], residuals: Optional[list] = None,
           dtype=torch.float64) -> torch.Tensor:
    """-> [len(tokens), vocab].  ``residuals`` (a list) receives the stream after every layer."""
    sd = {k: (v.to(dtype) if v.dtype.is_floating_point else v) for k, v in weights.items()}
    eps, groups = cfg["norm"]["eps"], cfg["norm"]["groups"]
    x = sd["embed"][torch.tensor(tokens)]
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        w = {k[len(p) + 4:]: v for k, v in sd.items() if k.startswith(p + "mix.")}
        a = group_norm(x, sd[p + "norm1"], groups, eps)
        a = a + causal_conv(a, sd[p + "canon1"])
        if layer["type"] == "delta":
            y = delta_mixer(a, w, layer["mixer"], eps)
        elif layer["type"] == "parallel":
            y = parallel_mixer(a, w, layer["mixer"], eps)
        else:
            raise ValueError(layer["type"])
        x = x + sd[p + "ls1"] * group_norm(y, sd[p + "norm1b"], groups, eps)
        if layer.get("mlp") is not None:
            b = group_norm(x, sd[p + "norm2"], groups, eps)
            b = b + causal_conv(b, sd[p + "canon2"])
            y = experts_ff(b, {k[len(p) + 4:]: v for k, v in sd.items() if k.startswith(p + "mlp.")}, layer["mlp"])
            x = x + sd[p + "ls2"] * group_norm(y, sd[p + "norm2b"], groups, eps)
        if residuals is not None:
            residuals.append(x.clone())
    x = group_norm(x, sd["final.norm"], groups, eps)
    return x @ sd["embed"].t()

"""RMSNorm, rotary embedding and gated activation layers backed by the HIP operators.

Each layer keeps the reference's two entry points: ``forward`` (native kernel) and
``_forward`` (plain PyTorch, the reference's own test oracle for the kernel):
vllm/model_executor/layers/layernorm.py:10-65, rotary_embedding.py:36-141,
activation.py:15-44.
"""
import math
from typing import Optional, Tuple, Union

import torch
import torch.nn as nn
import torch.nn.functional as F

from ... import _C


class RMSNorm(nn.Module):
    def __init__(self, hidden_size: int, eps: float = 1e-6) -> None:
        super().__init__()
        self.weight = nn.Parameter(torch.ones(hidden_size))
        self.variance_epsilon = eps

    def _forward(self, x: torch.Tensor, residual: Optional[torch.Tensor] = None):
        orig_dtype = x.dtype
        x = x.to(torch.float32)
        if residual is not None:
            x = x + residual.to(torch.float32)
            residual = x.to(orig_dtype)
        variance = x.pow(2).mean(dim=-1, keepdim=True)
        x = x * torch.rsqrt(variance + self.variance_epsilon)
        x = x.to(orig_dtype) * self.weight
        return x if residual is None else (x, residual)

    def forward(self, x: torch.Tensor, residual: Optional[torch.Tensor] = None
                ) -> Union[torch.Tensor, Tuple[torch.Tensor, torch.Tensor]]:
        if residual is not None:
            _C.ops.fused_add_rms_norm(x, residual, self.weight.data, self.variance_epsilon)
            return x, residual
        out = torch.empty_like(x)
        _C.ops.rms_norm(out, x, self.weight.data, self.variance_epsilon)
        return out


class RotaryEmbedding(nn.Module):
    """cos / sin table per position, applied in place to q and k."""

    def __init__(self, head_size: int, rotary_dim: int, max_position_embeddings: int, base: float,
                 is_neox_style: bool, dtype: torch.dtype) -> None:
        super().__init__()
        self.head_size = head_size
        self.rotary_dim = rotary_dim
        self.is_neox_style = is_neox_style
        inv_freq = 1.0 / (base ** (torch.arange(0, rotary_dim, 2, dtype=torch.float) / rotary_dim))
        t = torch.arange(max_position_embeddings, dtype=torch.float)
        freqs = torch.einsum("i,j -> ij", t, inv_freq)
        cache = torch.cat((freqs.cos(), freqs.sin()), dim=-1).to(dtype)      # [max_pos, rot_dim]
        self.register_buffer("cos_sin_cache", cache, persistent=False)

    def _forward(self, positions: torch.Tensor, query: torch.Tensor, key: torch.Tensor):
        """PyTorch restatement (rotary_embedding.py:88-122), fp32 products rounded once."""
        shape_q, shape_k = query.shape, key.shape
        cos_sin = self.cos_sin_cache[positions.flatten()].float()
        cos, sin = cos_sin.chunk(2, dim=-1)
        cos, sin = cos.unsqueeze(1), sin.unsqueeze(1)

        def rot(x):
            x = x.reshape(cos.shape[0], -1, self.head_size).float()
            xr, xp = x[..., :self.rotary_dim], x[..., self.rotary_dim:]
            if self.is_neox_style:
                x1, x2 = xr.chunk(2, dim=-1)
                o = torch.cat((x1 * cos - x2 * sin, x2 * cos + x1 * sin), dim=-1)
            else:
                x1, x2 = xr[..., ::2], xr[..., 1::2]
                o = torch.stack((x1 * cos - x2 * sin, x2 * cos + x1 * sin), dim=-1).flatten(-2)
            return torch.cat((o, xp), dim=-1)

        return rot(query).to(query.dtype).reshape(shape_q), rot(key).to(key.dtype).reshape(shape_k)

    def forward(self, positions: torch.Tensor, query: torch.Tensor, key: torch.Tensor):
        _C.ops.rotary_embedding(positions.flatten(), query, key, self.head_size, self.cos_sin_cache,
                                self.is_neox_style)
        return query, key

    def fusable_with_cache_write(self, dtype: torch.dtype) -> bool:
        """Whether ``ops.rotary_embedding_and_cache`` takes this geometry: the rotated part (its halves for
        the neox pairing), the rest of the head and the head itself span whole 16-byte vectors."""
        n = 16 // torch.empty((), dtype=dtype).element_size()
        rot = self.rotary_dim // 2 if self.is_neox_style else self.rotary_dim
        return (self.rotary_dim % 2 == 0 and rot % n == 0 and (self.head_size - self.rotary_dim) % n == 0
                and self.head_size % n == 0)


class SiluAndMul(nn.Module):
    def _forward(self, x: torch.Tensor) -> torch.Tensor:
        d = x.shape[-1] // 2
        return F.silu(x[..., :d]) * x[..., d:]

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        d = x.shape[-1] // 2
        out = torch.empty(x.shape[:-1] + (d,), dtype=x.dtype, device=x.device)
        _C.ops.silu_and_mul(out, x)
        return out


class ScalarRMSNorm(nn.Module):
    """RMS norm with ONE gain for all coordinates, applied to a sublayer's OUTPUT and added to an fp32
    residual stream: residual += y / sqrt(mean(y^2) + eps) * g.  The gain is kept in fp32."""

    def __init__(self, eps: float = 1e-6) -> None:
        super().__init__()
        self.weight = nn.Parameter(torch.ones(1, dtype=torch.float32), requires_grad=False)
        self.variance_epsilon = eps

    def _forward(self, residual: torch.Tensor, y: torch.Tensor) -> torch.Tensor:
        y = y.float()
        return residual + y * torch.rsqrt(y.pow(2).mean(-1, keepdim=True) + self.variance_epsilon) * self.weight

    def add_to(self, residual: torch.Tensor, y: torch.Tensor, cast_out: Optional[torch.Tensor] = None) -> None:
        """In place on ``residual``; ``cast_out`` receives the new residual in the activation dtype (the next
        sublayer's input)."""
        _C.mixer_ops.scalar_norm_add(residual, y, self.weight.data, self.variance_epsilon, cast_out)

    def forward(self, x: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
        """The model's final norm: fp32 stream in, activations out."""
        out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
        _C.mixer_ops.scalar_norm(out, x, self.weight.data, self.variance_epsilon)
        return out


class OffsetRMSNorm(nn.Module):
    """RMS norm of an fp32 residual stream with a per-channel weight stored as a difference from ``offset``:
    out = x / sqrt(mean(x^2) + eps) * (offset + w).  ``add_norm`` first sums sublayer outputs into the stream
    (x += a + b + c, the addends summed first), so a layer whose sublayers run side by side on one norm costs one
    pass over the stream per layer.  The weight is kept in fp32."""

    def __init__(self, width: int, eps: float = 1e-6, offset: float = 1.0) -> None:
        super().__init__()
        self.weight = nn.Parameter(torch.zeros(width, dtype=torch.float32), requires_grad=False)
        self.variance_epsilon, self.offset = eps, float(offset)

    def _forward(self, x: torch.Tensor) -> torch.Tensor:
        x = x.float()
        return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + self.variance_epsilon) * (self.offset + self.weight)

    def add_norm(self, residual: torch.Tensor, out_dtype: torch.dtype, a: Optional[torch.Tensor] = None,
                 b: Optional[torch.Tensor] = None, c: Optional[torch.Tensor] = None) -> torch.Tensor:
        """``residual`` fp32, updated in place; a, b: sublayer outputs in ``out_dtype``; c: an fp32 one."""
        out = torch.empty(residual.shape, dtype=out_dtype, device=residual.device)
        _C.mixer_ops.stream_add_norm(residual, self.weight.data, self.offset, self.variance_epsilon, out, a, b, c)
        return out

    def forward(self, x: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
        return self.add_norm(x, out_dtype)


class GroupRMSNorm(nn.Module):
    """RMS norm in groups of channels: the row is cut into ``groups`` equal runs, every run is divided by its own
    sqrt(mean(run^2) + eps), and the row is multiplied by a per-channel weight (kept in fp32).  Reads an fp32 stream.
    For layers that norm a sublayer's input AND its output, ``add_norm`` takes the sublayer's output through this
    norm (as the norm AFTER the sublayer) into the stream, times an optional per-channel layer scale, and writes the
    norm of the new stream that the next sublayer reads -- one launch."""

    def __init__(self, width: int, groups: int = 1, eps: float = 1e-6) -> None:
        super().__init__()
        if width % groups != 0:
            raise ValueError(f"a norm over {width} channels cannot be cut into {groups} equal groups")
        self.weight = nn.Parameter(torch.ones(width, dtype=torch.float32), requires_grad=False)
        self.groups, self.variance_epsilon = int(groups), eps

    def _forward(self, x: torch.Tensor) -> torch.Tensor:
        parts = x.float().unflatten(-1, (self.groups, -1))
        parts = parts * torch.rsqrt(parts.pow(2).mean(-1, keepdim=True) + self.variance_epsilon)
        return parts.flatten(-2) * self.weight

    def forward(self, stream: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
        out = torch.empty(stream.shape, dtype=out_dtype, device=stream.device)
        _C.mixer_ops.group_norm_add(stream, self.groups, self.variance_epsilon, weight=self.weight.data, out=out)
        return out

    def add_norm(self, stream: torch.Tensor, y: torch.Tensor, layer_scale: Optional[torch.Tensor],
                 next_norm: Optional["GroupRMSNorm"], out_dtype: torch.dtype, y2: Optional[torch.Tensor] = None,
                 s1: float = 1.0, s2: float = 1.0) -> Optional[torch.Tensor]:
        """stream (fp32, in place) += layer_scale * self(s1 * y + s2 * y2);  -> next_norm(stream) in ``out_dtype``
        (None without a next norm)."""
        out = None
        if next_norm is not None:
            assert next_norm.groups == self.groups and next_norm.variance_epsilon == self.variance_epsilon
            out = torch.empty(stream.shape, dtype=out_dtype, device=stream.device)
        _C.mixer_ops.group_norm_add(stream, self.groups, self.variance_epsilon, y, self.weight.data, layer_scale, y2,
                                    s1, s2, None if next_norm is None else next_norm.weight.data, out)
        return out


class CausalConvResidual(nn.Module):
    """A sublayer's input plus its own short causal convolution over time, per channel, no bias, no activation:
    out_t = x_t + sum_j taps[:, j] x_(t - T + 1 + j), rows before the sequence's start counting as zeros.  The last
    T - 1 inputs of every sequence are part of its state (``state_shape`` per slot, fp32)."""

    def __init__(self, channels: int, taps: int) -> None:
        super().__init__()
        self.channels, self.num_taps = channels, int(taps)
        self.taps = nn.Parameter(torch.zeros(channels, taps, dtype=torch.float32), requires_grad=False)

    def state_shape(self) -> Tuple[int, int]:
        return (self.num_taps - 1, self.channels)

    def forward(self, x: torch.Tensor, state: torch.Tensor, md, out_dtype: torch.dtype) -> torch.Tensor:
        out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
        _C.mixer_ops.causal_conv(out, x, self.taps.data, state, md.ragged, silu=False, residual=True)
        return out


class DynamicTanhNorm(nn.Module):
    """Element-wise norm without statistics of the row: out = tanh(alpha * x) * w + b, one number alpha, per-channel
    w and b, all kept in fp32; reads an fp32 stream and writes activations.  ``gated_add_norm`` first takes a
    sublayer's output into the stream through its gate (stream += mult * y * sigmoid(gate)) and, given the history of
    layer outputs with the layer's depth weights, files the sum and replaces the stream by the weighted mix of all
    entries, all in the one pass that also writes the norm."""

    def __init__(self, width: int) -> None:
        super().__init__()
        self.alpha = nn.Parameter(torch.ones(1, dtype=torch.float32), requires_grad=False)
        self.weight = nn.Parameter(torch.ones(width, dtype=torch.float32), requires_grad=False)
        self.bias = nn.Parameter(torch.zeros(width, dtype=torch.float32), requires_grad=False)

    def _forward(self, x: torch.Tensor) -> torch.Tensor:
        return torch.tanh(self.alpha * x.float()) * self.weight + self.bias

    def gated_add_norm(self, stream: torch.Tensor, out_dtype: torch.dtype, y: Optional[torch.Tensor] = None,
                       gate: Optional[torch.Tensor] = None, mult: float = 1.0,
                       history: Optional[torch.Tensor] = None,
                       depth_weights: Optional[torch.Tensor] = None) -> torch.Tensor:
        out = torch.empty(stream.shape, dtype=out_dtype, device=stream.device)
        _C.mixer_ops.gated_stream_step(stream, y, gate, mult, history, depth_weights,
                                       (self.alpha.data, self.weight.data, self.bias.data), out)
        return out

    def forward(self, x: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
        return self.gated_add_norm(x, out_dtype)

    def load_named(self, state: dict, name: str) -> None:
        self.weight.data.copy_(state[name].float())
        self.alpha.data.copy_(state[name + ".alpha"].float().reshape(1))
        self.bias.data.copy_(state[name + ".b"].float())


class PolyNorm(nn.Module):
    """Activation a U(z) + b U(z^2) + c U(z^3) + e with U(u) = u / sqrt(mean(u^2) + eps) over a row and the powers
    taken element by element; the four numbers are one fp32 parameter."""

    def __init__(self, eps: float) -> None:
        super().__init__()
        self.coef = nn.Parameter(torch.tensor([1.0, 0.0, 0.0, 0.0], dtype=torch.float32), requires_grad=False)
        self.eps = eps

    def _forward(self, z: torch.Tensor) -> torch.Tensor:
        z = z.float()

        def unit(u):
            return u * torch.rsqrt(u.pow(2).mean(-1, keepdim=True) + self.eps)
        c = self.coef
        return c[0] * unit(z) + c[1] * unit(z * z) + c[2] * unit(z * z * z) + c[3]

    def forward(self, z: torch.Tensor) -> torch.Tensor:
        """z: a 2-D view (a column range of a merged projection is fine)."""
        out = torch.empty(z.shape, dtype=z.dtype, device=z.device)
        _C.mixer_ops.poly_norm(out, z, self.coef.data, self.eps)
        return out


def rotary_frequencies(rot_dims: int, base: float) -> torch.Tensor:
    """fp32 [rot_dims / 2]: f_i = base^(-2i / rot_dims), worked out in double precision, rounded once."""
    return torch.tensor([float(base) ** (-2.0 * i / rot_dims) for i in range(rot_dims // 2)],
                        dtype=torch.float64).to(torch.float32)


def scaled_rotary_frequencies(rot_dims: int, base: float, scaling: Optional[dict] = None) -> torch.Tensor:
    """fp32 [rot_dims / 2]: f_i = base^(-2i / rot_dims), with long waves slowed down as Llama 3.1 does it
    (``scaling``: factor, low, high, original): a wavelength below original / high keeps f, one above original / low
    gets f / factor, between the two the mix (1 - s) f / factor + s f with s = (original / wavelength - low) /
    (high - low).  Worked out in double precision, rounded once."""
    out = []
    for i in range(rot_dims // 2):
        f = float(base) ** (-2.0 * i / rot_dims)
        if scaling:
            wavelength = 2.0 * math.pi / f
            original, low, high = scaling["original"], scaling["low"], scaling["high"]
            if wavelength < original / high:
                pass
            elif wavelength > original / low:
                f /= scaling["factor"]
            else:
                s = (original / wavelength - low) / (high - low)
                f = (1.0 - s) * f / scaling["factor"] + s * f
        out.append(f)
    return torch.tensor(out, dtype=torch.float64).to(torch.float32)


class ClampedGLU(nn.Module):
    """Gated activation with limits: x = gate | up;  g = min(gate, limit), u = clamp(up, -limit, limit);
    out = g * sigmoid(alpha * g) * (u + shift).  alpha = 1.702 makes g sigmoid(alpha g) the sigmoid form of gelu."""

    def __init__(self, alpha: float = 1.702, limit: float = math.inf, shift: float = 1.0) -> None:
        super().__init__()
        self.alpha, self.limit, self.shift = float(alpha), float(limit), float(shift)

    def _forward(self, x: torch.Tensor) -> torch.Tensor:
        d = x.shape[-1] // 2
        g = x[..., :d].float().clamp(max=self.limit)
        u = x[..., d:].float().clamp(-self.limit, self.limit)
        return (g * torch.sigmoid(self.alpha * g) * (u + self.shift)).to(x.dtype)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        out = torch.empty(x.shape[0], x.shape[1] // 2, dtype=x.dtype, device=x.device)
        _C.mixer_ops.clamped_glu(out, x, self.alpha, self.limit, self.shift)
        return out


class ReluSquared(nn.Module):
    def _forward(self, x: torch.Tensor) -> torch.Tensor:
        return torch.relu(x).pow(2)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
        _C.mixer_ops.relu2(out, x)
        return out

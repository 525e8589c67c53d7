"""Token mixers with a per-sequence recurrent state: delta-rule layers and the short causal convolution
in front of them.

A layer's state lives in the worker's state pools (``worker/cache_engine.py``), one slot per live sequence:
``state_shapes()`` names what the layer needs per slot, ``forward`` receives the allocated tensors.  All of a
layer's projections of the same input are one GEMM; everything that enters the recurrence besides the
projections (decays, step sizes, gates, unit norms, the state itself) is fp32 inside the kernels.

Delta rule, per head, S [key size, value size] (keys index rows):
  ``ChannelDeltaMixer``   S <- diag(g) S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q
                          g = exp(-exp(A_log) softplus(low-rank(h) + dt_bias)) per head and key channel
  ``GatedDeltaMixer``     the same rule with ONE decay per head: g = exp(-exp(A_log) softplus(W_a h + dt_bias));
                          the gate on the normed output is silu(W_g h)
  ``GeneralDeltaMixer``   S <- diag(w) S - (a * u)(u^T S) + k v^T;  o = S^T r,  u = k / |k|
                          w = exp(-e^(-1/2) sigmoid(low-rank-tanh(h) + w0)),  a = sigmoid(W_a h + b)

Linear attention, per head, S [key size, value size]:
  ``LightningMixer``      S <- decay_h S + k v^T;  o = S^T q,  q, k, v = silu of their projections; the heads'
                          outputs are normed together, gated by a sigmoid and projected
  ``GatedLinearAttentionMixer``  S <- diag(a) S + k v^T;  o = S^T q dim^(-1/2),  a = sigmoid(low-rank(h) + b)^(1 / tau)
                          per head and key channel; each head's output is normed with a weight shared by the
                          heads, gated by silu(gate) and projected
"""
from typing import Dict, List, Sequence, Tuple

import torch
import torch.nn as nn

from ... import _C
from ..input_metadata import InputMetadata
from .linear import ColumnParallelLinear, MergedColumnParallelLinear, RowParallelLinear


def _f32_param(*shape: int) -> nn.Parameter:
    return nn.Parameter(torch.zeros(*shape, dtype=torch.float32), requires_grad=False)


class ChannelDeltaMixer(nn.Module):
    def __init__(self, width: int, heads: int, kv_heads: int, dim: int, vdim: int, conv_taps: int, decay_rank: int,
                 gate_rank: int, eps: float, dtype: torch.dtype, linear_method=None) -> None:
        super().__init__()
        assert heads % kv_heads == 0
        self.heads, self.kv_heads, self.dim, self.vdim, self.taps, self.eps = heads, kv_heads, dim, vdim, conv_taps, eps
        self.conv_channels = 2 * kv_heads * dim + heads * vdim          # q | k | v
        # q | k | v | beta | decay (low rank, first factor) | gate (low rank, first factor)
        self.in_sizes = [kv_heads * dim, kv_heads * dim, heads * vdim, heads, decay_rank, gate_rank]
        self.in_proj = MergedColumnParallelLinear(width, self.in_sizes, False, dtype, linear_method)
        self.decay_up = ColumnParallelLinear(decay_rank, heads * dim, False, dtype, linear_method)
        self.gate_up = ColumnParallelLinear(gate_rank, heads * vdim, False, dtype, linear_method)
        self.o_proj = RowParallelLinear(heads * vdim, width, False, dtype, linear_method)
        self.conv_taps = _f32_param(self.conv_channels, conv_taps)
        self.dt_bias = _f32_param(heads * dim)
        self.a_log = _f32_param(heads)
        self.out_norm = nn.Parameter(torch.ones(vdim, dtype=torch.float32), requires_grad=False)

    def state_shapes(self) -> List[Tuple[int, ...]]:
        """Per slot: the convolution's last inputs, the delta-rule state."""
        return [(self.taps - 1, self.conv_channels), (self.heads, self.dim, self.vdim)]

    def forward(self, h: torch.Tensor, state: List[torch.Tensor], md: InputMetadata) -> torch.Tensor:
        conv_state, rule_state = state
        batch = md.ragged
        rows = h.shape[0]
        proj = self.in_proj(h)
        c = self.conv_channels
        beta_pre = proj[:, c:c + self.heads]
        lo = c + self.heads
        decay_pre = self.decay_up(proj[:, lo:lo + self.in_sizes[4]])
        gate_pre = self.gate_up(proj[:, lo + self.in_sizes[4]:])
        qkv = torch.empty(rows, c, dtype=torch.float32, device=h.device)
        _C.mixer_ops.short_conv(qkv, proj[:, :c], self.conv_taps.data, conv_state, batch)
        o = torch.empty(rows, self.heads * self.vdim, dtype=torch.float32, device=h.device)
        _C.mixer_ops.channel_delta(o, qkv, beta_pre, decay_pre, self.dt_bias.data, self.a_log.data, rule_state, batch,
                                   self.heads, self.kv_heads, self.dim, self.vdim)
        gated = torch.empty(rows, self.heads * self.vdim, dtype=h.dtype, device=h.device)
        _C.mixer_ops.head_norm_gate(gated, o, gate_pre, self.out_norm.data, False, self.eps, self.heads, self.vdim)
        return self.o_proj(gated)

    def load_named(self, w: Dict[str, torch.Tensor]) -> None:
        """``w``: the layer's checkpoint tensors by their short names (q, q.conv, k, ..., o)."""
        dev = self.dt_bias.device
        self.in_proj.weight.data.copy_(torch.cat([w["q"], w["k"], w["v"], w["b"], w["a1"], w["g1"]], 0))
        self.decay_up.weight.data.copy_(w["a2"])
        self.gate_up.weight.data.copy_(w["g2"])
        self.o_proj.weight.data.copy_(w["o"])
        self.conv_taps.data.copy_(torch.cat([w["q.conv"], w["k.conv"], w["v.conv"]], 0).float().to(dev))
        self.dt_bias.data.copy_(w["dt_bias"].float())
        self.a_log.data.copy_(w["A_log"].float())
        self.out_norm.data.copy_(w["norm"].float())


class GatedDeltaMixer(nn.Module):
    """Delta rule with a gate beta and one decay per head (see the module's docstring).  q | k | v | beta | decay |
    output gate are one GEMM of the layer's input; q, k, v pass a short causal convolution per channel and silu; q and
    k are made unit vectors per head inside the kernel (q also times dim^-1/2); value head h reads q / k head
    h // (heads / kv_heads).  Each head's output gets an RMS norm over its value channels with ONE weight [vdim]
    shared by the heads, times silu(gate), then the output projection."""

    def __init__(self, width: int, heads: int, kv_heads: int, dim: int, vdim: int, conv_taps: int, eps: float,
                 dtype: torch.dtype, linear_method=None) -> None:
        super().__init__()
        assert heads % kv_heads == 0
        self.heads, self.kv_heads, self.dim, self.vdim, self.taps, self.eps = heads, kv_heads, dim, vdim, conv_taps, eps
        self.conv_channels = 2 * kv_heads * dim + heads * vdim          # q | k | v
        self.in_sizes = [kv_heads * dim, kv_heads * dim, heads * vdim, heads, heads, heads * vdim]
        self.in_proj = MergedColumnParallelLinear(width, self.in_sizes, False, dtype, linear_method)
        self.o_proj = RowParallelLinear(heads * vdim, width, False, dtype, linear_method)
        self.conv_taps = _f32_param(self.conv_channels, conv_taps)
        self.dt_bias = _f32_param(heads)
        self.a_log = _f32_param(heads)
        self.out_norm = nn.Parameter(torch.ones(vdim, dtype=torch.float32), requires_grad=False)

    def state_shapes(self) -> List[Tuple[int, ...]]:
        """Per slot: the convolution's last inputs, the delta-rule state."""
        return [(self.taps - 1, self.conv_channels), (self.heads, self.dim, self.vdim)]

    def forward(self, h: torch.Tensor, state: List[torch.Tensor], md: InputMetadata) -> torch.Tensor:
        conv_state, rule_state = state
        batch = md.ragged
        rows, c, H = h.shape[0], self.conv_channels, self.heads
        proj = self.in_proj(h)
        qkv = torch.empty(rows, c, dtype=torch.float32, device=h.device)
        _C.mixer_ops.causal_conv(qkv, proj[:, :c], self.conv_taps.data, conv_state, batch, silu=True, residual=False)
        o = torch.empty(rows, H * self.vdim, dtype=torch.float32, device=h.device)
        _C.mixer_ops.gated_delta(o, qkv, proj[:, c:c + H], proj[:, c + H:c + 2 * H], self.dt_bias.data, self.a_log.data,
                                 rule_state, batch, H, self.kv_heads, self.dim, self.vdim)
        gated = torch.empty(rows, H * self.vdim, dtype=h.dtype, device=h.device)
        _C.mixer_ops.head_norm_gate(gated, o, proj[:, c + 2 * H:], self.out_norm.data, False, self.eps, H, self.vdim,
                                    gate_silu=True)
        return self.o_proj(gated)

    def load_named(self, w: Dict[str, torch.Tensor]) -> None:
        """``w``: q, q.conv, k, k.conv, v, v.conv, b, a, dt_bias, A_log, g, norm, o."""
        self.in_proj.weight.data.copy_(torch.cat([w["q"], w["k"], w["v"], w["b"], w["a"], w["g"]], 0))
        self.o_proj.weight.data.copy_(w["o"])
        self.conv_taps.data.copy_(torch.cat([w["q.conv"], w["k.conv"], w["v.conv"]], 0).float())
        self.dt_bias.data.copy_(w["dt_bias"].float())
        self.a_log.data.copy_(w["A_log"].float())
        self.out_norm.data.copy_(w["norm"].float())


class GeneralDeltaMixer(nn.Module):
    def __init__(self, width: int, heads: int, dim: int, decay_rank: int, eps: float, dtype: torch.dtype,
                 linear_method=None) -> None:
        super().__init__()
        self.heads, self.dim, self.eps = heads, dim, eps
        size = heads * dim
        self.size = size
        # r | k | v | gate | removal rate | decay (low rank, first factor)
        self.in_sizes = [size, size, size, size, size, decay_rank]
        self.in_proj = MergedColumnParallelLinear(width, self.in_sizes, False, dtype, linear_method)
        self.decay_up = ColumnParallelLinear(decay_rank, size, False, dtype, linear_method)
        self.o_proj = RowParallelLinear(size, width, False, dtype, linear_method)
        self.w0 = _f32_param(size)
        self.rate_bias = _f32_param(size)
        self.out_norm = nn.Parameter(torch.ones(size, dtype=torch.float32), requires_grad=False)

    def state_shapes(self) -> List[Tuple[int, ...]]:
        return [(self.heads, self.dim, self.dim)]

    def forward(self, h: torch.Tensor, state: List[torch.Tensor], md: InputMetadata) -> torch.Tensor:
        batch = md.ragged
        rows, n = h.shape[0], self.size
        proj = self.in_proj(h)
        decay_pre = self.decay_up(torch.tanh(proj[:, 5 * n:]))
        o = torch.empty(rows, n, dtype=torch.float32, device=h.device)
        _C.mixer_ops.general_delta(o, proj[:, :n], proj[:, n:2 * n], proj[:, 2 * n:3 * n], decay_pre, self.w0.data,
                                   proj[:, 4 * n:5 * n], self.rate_bias.data, state[0], batch, self.heads, self.dim)
        gated = torch.empty(rows, n, dtype=h.dtype, device=h.device)
        _C.mixer_ops.head_norm_gate(gated, o, proj[:, 3 * n:4 * n], self.out_norm.data, True, self.eps, self.heads,
                                    self.dim)
        return self.o_proj(gated)

    def load_named(self, w: Dict[str, torch.Tensor]) -> None:
        self.in_proj.weight.data.copy_(torch.cat([w["r"], w["k"], w["v"], w["g"], w["a"], w["w1"]], 0))
        self.decay_up.weight.data.copy_(w["w2"])
        self.o_proj.weight.data.copy_(w["o"])
        self.w0.data.copy_(w["w0"].float())
        self.rate_bias.data.copy_(w["a.b"].float())
        self.out_norm.data.copy_(w["norm"].float())


class LightningMixer(nn.Module):
    """Linear attention with one constant decay per head.  q | k | v | gate are one GEMM of the layer's input; the
    recurrence runs in fp32 on the silu of q, k, v (chunks of 32 tokens as matrix products); the concatenated heads
    get ONE RMS norm over all of them (weight [heads * vdim]), times sigmoid(gate), then the output projection."""

    def __init__(self, width: int, heads: int, dim: int, vdim: int, decay: Sequence[float], eps: float,
                 dtype: torch.dtype, linear_method=None) -> None:
        super().__init__()
        assert len(decay) == heads
        self.heads, self.dim, self.vdim, self.eps = heads, dim, vdim, eps
        self.in_sizes = [heads * dim, heads * dim, heads * vdim, heads * vdim]
        self.in_proj = MergedColumnParallelLinear(width, self.in_sizes, False, dtype, linear_method)
        self.o_proj = RowParallelLinear(heads * vdim, width, False, dtype, linear_method)
        # a constant of the config, not a weight
        self.register_buffer("decay", torch.tensor([float(d) for d in decay], dtype=torch.float64).to(torch.float32),
                             persistent=False)
        self.out_norm = nn.Parameter(torch.ones(heads * vdim, dtype=torch.float32), requires_grad=False)

    def state_shapes(self) -> List[Tuple[int, ...]]:
        return [(self.heads, self.dim, self.vdim)]

    def forward(self, h: torch.Tensor, state: List[torch.Tensor], md: InputMetadata) -> torch.Tensor:
        rows = h.shape[0]
        proj = self.in_proj(h)
        nk, nv = self.heads * self.dim, self.heads * self.vdim
        o = torch.empty(rows, nv, dtype=torch.float32, device=h.device)
        _C.mixer_ops.lightning(o, proj[:, :nk], proj[:, nk:2 * nk], proj[:, 2 * nk:2 * nk + nv], self.decay,
                               state[0], md.ragged, self.heads, self.dim, self.vdim)
        gated = torch.empty(rows, nv, dtype=h.dtype, device=h.device)
        # one "head" of heads * vdim channels: the norm runs over all heads together
        _C.mixer_ops.head_norm_gate(gated, o, proj[:, 2 * nk + nv:], self.out_norm.data, True, self.eps, 1, nv)
        return self.o_proj(gated)

    def load_named(self, w: Dict[str, torch.Tensor]) -> None:
        self.in_proj.weight.data.copy_(torch.cat([w["q"], w["k"], w["v"], w["g"]], 0))
        self.o_proj.weight.data.copy_(w["o"])
        self.out_norm.data.copy_(w["norm"].float())


class GatedLinearAttentionMixer(nn.Module):
    """Linear attention with a data-dependent decay per head and key channel, a_t = sigmoid(z_t)^(1 / tau) with z a
    low-rank projection of the layer's input plus a bias.  q | k | v | gate | first decay factor (| ``extra_out``
    more columns for the caller, e.g. a gate on the layer's output) are one GEMM; the decay's logarithm, the
    recurrence and the output norm are fp32.  Each head's output gets an RMS norm over its value channels with ONE
    weight [vdim] shared by the heads, times silu(gate), then the output projection.  Built with ``project=False``
    the mixer owns neither the input nor the output projection: a layer that runs it beside another mixer on ONE
    input GEMM hands the column ranges to ``core`` and projects the result itself."""

    def __init__(self, width: int, heads: int, dim: int, vdim: int, decay_rank: int, tau: float, eps: float,
                 dtype: torch.dtype, linear_method=None, extra_out: int = 0, project: bool = True) -> None:
        super().__init__()
        self.heads, self.dim, self.vdim, self.tau, self.eps = heads, dim, vdim, float(tau), eps
        self.in_sizes = [heads * dim, heads * dim, heads * vdim, heads * vdim, decay_rank] + \
            ([extra_out] if extra_out else [])
        self.in_proj = self.o_proj = None
        if project:
            self.in_proj = MergedColumnParallelLinear(width, self.in_sizes, bool(extra_out), dtype, linear_method)
            self.o_proj = RowParallelLinear(heads * vdim, width, False, dtype, linear_method)
        self.decay_up = ColumnParallelLinear(decay_rank, heads * dim, False, dtype, linear_method)
        self.decay_bias = _f32_param(heads * dim)
        self.out_norm = nn.Parameter(torch.ones(vdim, dtype=torch.float32), requires_grad=False)

    def state_shapes(self) -> List[Tuple[int, ...]]:
        return [(self.heads, self.dim, self.vdim)]

    def forward(self, h: torch.Tensor, state: List[torch.Tensor], md: InputMetadata):
        """-> (output [rows, width], the ``extra_out`` columns of the input projection or None)."""
        proj = self.in_proj(h)
        nk, nv, rank = self.heads * self.dim, self.heads * self.vdim, self.in_sizes[4]
        lo = 2 * nk + 2 * nv
        gated = self.core(proj[:, :nk], proj[:, nk:2 * nk], proj[:, 2 * nk:2 * nk + nv], proj[:, 2 * nk + nv:lo],
                          proj[:, lo:lo + rank], state[0], md)
        extra = proj[:, lo + rank:] if len(self.in_sizes) > 5 else None
        return self.o_proj(gated), extra

    def core(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, gate: torch.Tensor, decay_low: torch.Tensor,
             state: torch.Tensor, md: InputMetadata) -> torch.Tensor:
        """q, k, v, gate, decay_low (the decay's first, low-rank factor): column ranges of ONE projection output.
        -> the normed, gated heads [rows, heads * vdim] in the activation dtype, before the output projection."""
        rows, nv = q.shape[0], self.heads * self.vdim
        decay_pre = self.decay_up(decay_low)
        o = torch.empty(rows, nv, dtype=torch.float32, device=q.device)
        _C.mixer_ops.gla(o, q, k, v, decay_pre, self.decay_bias.data, self.tau, self.dim ** -0.5, state, md.ragged,
                         self.heads, self.dim, self.vdim)
        gated = torch.empty(rows, nv, dtype=q.dtype, device=q.device)
        _C.mixer_ops.head_norm_gate(gated, o, gate, self.out_norm.data, False, self.eps, self.heads, self.vdim,
                                    gate_silu=True)
        return gated

    def load_named(self, w: Dict[str, torch.Tensor], extra: Dict[str, torch.Tensor] = None) -> None:
        """``w``: q, k, v, g, a1, a2, a2.b, norm, o; ``extra``: weight / bias of the ``extra_out`` columns.  A mixer
        without projections of its own takes a2, a2.b and norm."""
        if self.in_proj is not None:
            parts = [w["q"], w["k"], w["v"], w["g"], w["a1"]] + ([extra["weight"]] if extra else [])
            self.in_proj.weight.data.copy_(torch.cat(parts, 0))
            if extra:
                self.in_proj.bias.data.zero_()
                self.in_proj.bias.data[-extra["bias"].numel():].copy_(extra["bias"])
            self.o_proj.weight.data.copy_(w["o"])
        self.decay_up.weight.data.copy_(w["a2"])
        self.decay_bias.data.copy_(w["a2.b"].float())
        self.out_norm.data.copy_(w["norm"].float())

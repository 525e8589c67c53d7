"""Mixture-of-experts feed-forward layers.

``TableRoutedExperts``: no learned router -- a table [vocab, top] names each token id's experts, every chosen
expert weighs 1 / top.  An expert is down(gelu(up x)) with the exact (erf) gelu and no biases.  An optional
shared expert of the same form runs for every token and is added after a per-token sigmoid gate.

``GroupRoutedExperts``: a learned sigmoid router in fp32 with a selection bias that enters the choice but not the
weights, a choice limited to the best groups of neighbouring experts, weights normalised over the chosen experts
and scaled; an expert is down(relu(up x)^2); an optional shared expert of the same form is returned beside the
routed sum so that the caller's residual add can take both.  The same layer, by its options, is a SOFTMAX router
(``score="softmax"``: scores are the softmax over all experts), whose groups score their best expert
(``group_score="max"``), whose weights are the chosen scores as they are (``normalize=False``) and whose experts have
a gated hidden layer with limits (``activation="clamped_glu"``: g = min(gate x, limit), u = clamp(up x, +-limit),
g sigmoid(alpha g) (u + 1)).

Rows are grouped by expert on the device (a stable sort of the (row, choice) pairs by expert id, then a binary
search for every expert's first pair), so each expert's rows are one contiguous run and the host never waits.
"""
from typing import Dict, Optional, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F

from ... import _C
from .linear import ColumnParallelLinear, MergedColumnParallelLinear, RowParallelLinear


class TableRoutedExperts(nn.Module):
    def __init__(self, width: int, vocab: int, num_experts: int, top: int, ff: int, shared_ff: Optional[int],
                 dtype: torch.dtype, linear_method=None) -> None:
        super().__init__()
        self.width, self.num_experts, self.top, self.ff = width, num_experts, top, ff
        self.table = nn.Parameter(torch.zeros(vocab, top, dtype=torch.int32), requires_grad=False)
        self.up = nn.Parameter(torch.empty(num_experts, ff, width, dtype=dtype), requires_grad=False)
        self.down = nn.Parameter(torch.empty(num_experts, width, ff, dtype=dtype), requires_grad=False)
        self.shared_ff = shared_ff
        if shared_ff:
            # shared expert's up projection and its gate read the same input: one GEMM
            self.shared_in = MergedColumnParallelLinear(width, [shared_ff, 1], False, dtype, linear_method)
            self.shared_down = RowParallelLinear(shared_ff, width, False, dtype, linear_method)

    def route(self, token_ids: torch.Tensor):
        """-> (order [rows * top] int32: pair index row * top + choice, sorted by expert;
               expert_start [experts + 1] int32)."""
        experts = self.table.data.index_select(0, token_ids).view(-1)              # [rows * top]
        by_expert, order = torch.sort(experts, stable=True)
        # first sorted pair of every expert: no count ever travels to the host
        edges = torch.arange(self.num_experts + 1, dtype=experts.dtype, device=experts.device)
        start = torch.searchsorted(by_expert, edges).to(torch.int32)
        return order.to(torch.int32), start

    def forward(self, h: torch.Tensor, token_ids: torch.Tensor) -> torch.Tensor:
        """-> fp32 [rows, width]: the experts' sum is accumulated in fp32."""
        rows = h.shape[0]
        order, start = self.route(token_ids)
        out = torch.zeros(rows, self.width, dtype=torch.float32, device=h.device)
        _C.mixer_ops.expert_ffn(out, h, self.up.data, self.down.data, order, start, self.top, 1.0 / self.top)
        if self.shared_ff:
            both = self.shared_in(h)
            hidden = F.gelu(both[:, :self.shared_ff])
            shared = self.shared_down(hidden)
            out.addcmul_(torch.sigmoid(both[:, self.shared_ff:].float()), shared.float())
        return out

    def load_named(self, w: Dict[str, torch.Tensor]) -> None:
        self.table.data.copy_(w["table"].to(torch.int32))
        self.up.data.copy_(torch.stack([w[f"e{e}.up"] for e in range(self.num_experts)]))
        self.down.data.copy_(torch.stack([w[f"e{e}.down"] for e in range(self.num_experts)]))
        if self.shared_ff:
            self.shared_in.weight.data.copy_(torch.cat([w["shared.up"], w["shared.sg"]], 0))
            self.shared_down.weight.data.copy_(w["shared.down"])


def group_pairs_by_expert(experts: torch.Tensor, num_experts: int):
    """experts int32 [rows, top] -> (order int32 [rows * top]: pair indices row * top + choice grouped by expert,
    expert_start int32 [experts + 1]); one launch on the device."""
    return _C.mixer_ops.group_pairs(experts, num_experts)


class GroupRoutedExperts(nn.Module):
    def __init__(self, width: int, num_experts: int, top: int, ff: int, shared_ff: Optional[int], groups: int,
                 keep_groups: int, scale: float, dtype: torch.dtype, linear_method=None, score: str = "sigmoid",
                 group_score: str = "top2", normalize: bool = True, activation: str = "relu2",
                 limit: float = float("inf"), glu_alpha: float = 1.702) -> None:
        super().__init__()
        if score not in ("sigmoid", "softmax") or group_score not in ("top2", "max") or \
                activation not in ("relu2", "clamped_glu"):
            raise ValueError(f"unknown router score {score!r}, group score {group_score!r} or activation {activation!r}")
        if activation == "clamped_glu" and shared_ff:
            raise NotImplementedError("a shared expert with a gated hidden layer")
        self.softmax, self.group_best_one, self.normalize = score == "softmax", group_score == "max", bool(normalize)
        self.glu = (float(glu_alpha), float(limit), 1.0) if activation == "clamped_glu" else None
        if num_experts % groups != 0 or not (1 <= keep_groups <= groups) or keep_groups * (num_experts // groups) < top:
            raise ValueError(f"{num_experts} experts in {groups} groups with {keep_groups} kept cannot give {top} choices")
        self.width, self.num_experts, self.top, self.ff = width, num_experts, top, ff
        self.groups, self.keep_groups, self.scale = groups, keep_groups, float(scale)
        # the router is fp32 whatever the model's dtype
        self.router = nn.Parameter(torch.zeros(num_experts, width, dtype=torch.float32), requires_grad=False)
        self.correction = nn.Parameter(torch.zeros(num_experts, dtype=torch.float32), requires_grad=False)
        # a gated hidden layer: gate and up rows in runs of 16, as the fused kernel reads them (``mixer_ops.glu_rows``)
        self.up = nn.Parameter(torch.empty(num_experts, 32 * (-(-ff // 16)) if self.glu else ff, width, dtype=dtype),
                               requires_grad=False)
        self.down = nn.Parameter(torch.empty(num_experts, width, ff, dtype=dtype), requires_grad=False)
        self.shared_ff = shared_ff
        if shared_ff:
            self.shared_up = ColumnParallelLinear(width, shared_ff, False, dtype, linear_method)
            self.shared_down = RowParallelLinear(shared_ff, width, False, dtype, linear_method)

    def forward(self, h: torch.Tensor) -> Tuple[Optional[torch.Tensor], torch.Tensor]:
        """-> (shared expert's output in h's dtype or None, routed experts' weighted sum in fp32)."""
        # fp32 products with the fp32 router (the library's GEMM; no reduced-precision matrix mode is switched on)
        logits = torch.matmul(h.float(), self.router.data.t())
        chosen, weights = _C.mixer_ops.group_router(logits, self.correction.data, self.top, self.groups,
                                                    self.keep_groups, self.scale, self.softmax, self.group_best_one,
                                                    self.normalize)
        order, start = group_pairs_by_expert(chosen, self.num_experts)
        out = torch.zeros(h.shape[0], self.width, dtype=torch.float32, device=h.device)
        _C.mixer_ops.expert_ffn(out, h, self.up.data, self.down.data, order, start, self.top, 1.0,
                                activation=_C.mixer_ops.ACT_RELU2, pair_weight=weights, glu=self.glu)
        shared = None
        if self.shared_ff:
            hidden = self.shared_up(h)
            act = torch.empty_like(hidden)
            _C.mixer_ops.relu2(act, hidden)
            shared = self.shared_down(act)
        return shared, out

    def load_named(self, w: Dict[str, torch.Tensor]) -> None:
        self.router.data.copy_(w["router"].float())
        if "correction" in w:
            self.correction.data.copy_(w["correction"].float())
        if self.glu:
            self.up.data.copy_(_C.mixer_ops.glu_rows(torch.stack([w[f"e{e}.gate"] for e in range(self.num_experts)]),
                                                     torch.stack([w[f"e{e}.up"] for e in range(self.num_experts)])))
        else:
            self.up.data.copy_(torch.stack([w[f"e{e}.up"] for e in range(self.num_experts)]))
        self.down.data.copy_(torch.stack([w[f"e{e}.down"] for e in range(self.num_experts)]))
        if self.shared_ff:
            self.shared_up.weight.data.copy_(w["shared.up"])
            self.shared_down.weight.data.copy_(w["shared.down"])

"""Lalasun: a decoder whose layers are listed one by one in its config.json, whose sublayer outputs enter the
residual stream through learned gates, and whose layers read a weighted mix of the outputs of all earlier layers.

Each entry of ``layers`` names the layer's token mixer -- ``latent_attention`` (keys and values of all heads from
one small latent per token plus a rotated key part shared by the heads, sliding window, sigmoid gate on the
heads' output), ``attention`` (grouped query heads with biased projections, rotary embedding on half-split pairs,
chunked mask, one more term in the softmax's denominator) or ``gla`` (gated linear attention with a decay per head
and key channel and a per-sequence fp32 state) -- with the mixer's sizes, and its feed-forward: ``dense``
(down(PolyNorm(up h))) or none.

A layer, with r = ``residual_mult`` and T = the element-wise tanh norm tanh(alpha u) w + b:
    h1 = T1(x);  y = x + r * mixer(h1) * sigmoid(G1 h1 + g1)
    h2 = T2(y);  X = y + r * ff(h2)    * sigmoid(G2 h2 + g2)
and what the next layer (or the output norm) receives is sum_j D[j] X_j over the embedding rows X_0 and the X of
every layer so far, with the layer's own weights D.  The stream and the history of X_j are fp32; a gate's
projection rides in the same GEMM as the sublayer's input projection, and the gated add, the filing into the
history, the depth mix and the next norm are one kernel.  The logits come from a matrix of their own.
Steps arrive in the ragged layout (``InputMetadata.ragged``): any mix of prompt portions and decoded tokens.

Per layer the worker allocates what ``cache_layout`` asks for: pages of latent rows or of keys / values for the
attention layers, per-sequence state slots for a gla layer.
"""
from typing import Dict, List, Optional

import torch
import torch.nn as nn

from ..input_metadata import InputMetadata
from ..layers.attention import CappedGatedAttention, LatentAttention
from ..layers.basic import DynamicTanhNorm, PolyNorm, rotary_frequencies
from ..layers.linear import LinearMethodBase, MergedColumnParallelLinear, RowParallelLinear
from ..layers.recurrent import GatedLinearAttentionMixer
from ..layers.sampler import Sampler, SamplingMetadata
from ..layers.vocab_parallel_embedding import VocabParallelEmbedding
from ..parallel_state import get_tensor_model_parallel_world_size

_MIXERS = ("latent_attention", "attention", "gla")


def normalize_config(raw: dict) -> dict:
    """The engine's generic geometry keys for a Lalasun config.json."""
    cfg = dict(raw)
    cfg["architecture"] = "lalasun"
    cfg["vocab_size"] = raw["vocab"]
    cfg["hidden_size"] = raw["width"]
    cfg["num_hidden_layers"] = len(raw["layers"])
    attn = [l["mixer"] for l in raw["layers"] if l["type"] in ("attention", "latent_attention")]
    cfg["num_attention_heads"] = attn[0]["heads"] if attn else 1
    cfg["num_key_value_heads"] = attn[0].get("kv_heads", attn[0]["heads"]) if attn else 1
    cfg.setdefault("max_position_embeddings", 1 << 20)       # angles come from fp32 positions: no table to outgrow
    cfg.setdefault("torch_dtype", "bfloat16")
    return cfg


def _set_bias_tail(linear: nn.Module, bias: torch.Tensor) -> None:
    """The last columns of a merged projection are the layer's output gate; only they have a bias."""
    linear.bias.data.zero_()
    linear.bias.data[-bias.numel():].copy_(bias)


class LalasunLatentAttention(nn.Module):
    def __init__(self, width: int, m: dict, eps: float, dtype, linear_method) -> None:
        super().__init__()
        h, d, dr, dv, rank = m["heads"], m["dim"], m["rot_dim"], m.get("vdim", m["dim"]), m["kv_rank"]
        rot = m["rot"]
        if rot["dims"] != dr:
            raise ValueError(f"latent_attention rotates its whole rotated part: rot.dims {rot['dims']} != rot_dim {dr}")
        # q | latent and shared key part | gate on the heads | gate on the layer's output: one GEMM
        self.sizes = [h * (d + dr), rank + dr, h * dv, width]
        self.in_proj = MergedColumnParallelLinear(width, self.sizes, True, dtype, linear_method)
        self.o_proj = RowParallelLinear(h * dv, width, False, dtype, linear_method)
        window = (m.get("mask") or {}).get("size", 0)
        self.attn = LatentAttention(h, d, dr, dv, rank, m["scale"], rotary_frequencies(dr, rot["base"]), eps, dtype,
                                    window)

    def forward(self, h: torch.Tensor, positions: torch.Tensor, cache: List[torch.Tensor], md: InputMetadata):
        proj = self.in_proj(h)
        a, b, c = self.sizes[0], self.sizes[0] + self.sizes[1], self.sizes[0] + self.sizes[1] + self.sizes[2]
        out = self.attn(proj[:, :a], proj[:, a:b], proj[:, b:c], positions, cache[0], md)
        return self.o_proj(out), proj[:, c:]

    def load_named(self, w: Dict[str, torch.Tensor], gate_w: torch.Tensor, gate_b: torch.Tensor) -> None:
        self.in_proj.weight.data.copy_(torch.cat([w["q"], w["dkv"], w["g"], gate_w], 0))
        _set_bias_tail(self.in_proj, gate_b)
        self.o_proj.weight.data.copy_(w["o"])
        self.attn.latent_norm.data.copy_(w["dkv.norm"].float())
        self.attn.load_up_projections(w["uk"], w["uv"])


class LalasunChunkedAttention(nn.Module):
    def __init__(self, width: int, m: dict, dtype, linear_method) -> None:
        super().__init__()
        h, d = m["heads"], m["dim"]
        g, dv = m.get("kv_heads", h), m.get("vdim", d)
        # q | k | v | gate on the layer's output: one GEMM, all with a bias
        self.sizes = [h * d, g * d, g * dv, width]
        self.in_proj = MergedColumnParallelLinear(width, self.sizes, True, dtype, linear_method)
        self.o_proj = RowParallelLinear(h * dv, width, True, dtype, linear_method)
        rot = m.get("rot")
        freqs = rotary_frequencies(rot["dims"], rot["base"]) if rot else None
        chunk = (m.get("mask") or {}).get("size", 0)
        self.attn = CappedGatedAttention(h, g, d, dv, m["scale"], 0.0, freqs, chunk=chunk, sink=True, pair_halves=True)

    def forward(self, h: torch.Tensor, positions: torch.Tensor, cache: List[torch.Tensor], md: InputMetadata):
        proj = self.in_proj(h)
        a, b, c = self.sizes[0], self.sizes[0] + self.sizes[1], self.sizes[0] + self.sizes[1] + self.sizes[2]
        out = self.attn(proj[:, :a], proj[:, a:b], proj[:, b:c], None, positions, cache[0], cache[1], md)
        return self.o_proj(out), proj[:, c:]

    def load_named(self, w: Dict[str, torch.Tensor], gate_w: torch.Tensor, gate_b: torch.Tensor) -> None:
        self.in_proj.weight.data.copy_(torch.cat([w["q"], w["k"], w["v"], gate_w], 0))
        self.in_proj.bias.data.copy_(torch.cat([w["q.b"], w["k.b"], w["v.b"], gate_b], 0))
        self.o_proj.weight.data.copy_(w["o"])
        self.o_proj.bias.data.copy_(w["o.b"])


class PolyNormMLP(nn.Module):
    """down(PolyNorm(up h)); the gate on the layer's output rides in the up-projection's GEMM."""

    def __init__(self, width: int, ff: int, eps: float, dtype, linear_method) -> None:
        super().__init__()
        self.ff = ff
        self.up = MergedColumnParallelLinear(width, [ff, width], True, dtype, linear_method)
        self.down = RowParallelLinear(ff, width, False, dtype, linear_method)
        self.act = PolyNorm(eps)

    def forward(self, h: torch.Tensor):
        proj = self.up(h)
        return self.down(self.act(proj[:, :self.ff])), proj[:, self.ff:]

    def load_named(self, w: Dict[str, torch.Tensor], gate_w: torch.Tensor, gate_b: torch.Tensor) -> None:
        self.up.weight.data.copy_(torch.cat([w["up"], gate_w], 0))
        _set_bias_tail(self.up, gate_b)
        self.down.weight.data.copy_(w["down"])
        self.act.coef.data.copy_(w["act"].float())


class LalasunLayer(nn.Module):
    def __init__(self, cfg: dict, index: int, dtype, linear_method) -> None:
        super().__init__()
        layer = cfg["layers"][index]
        width, eps, m = cfg["width"], cfg["norm"]["eps"], layer["mixer"]
        self.kind = layer["type"]
        if self.kind == "latent_attention":
            self.mix = LalasunLatentAttention(width, m, eps, dtype, linear_method)
        elif self.kind == "attention":
            self.mix = LalasunChunkedAttention(width, m, dtype, linear_method)
        elif self.kind == "gla":
            self.mix = GatedLinearAttentionMixer(width, m["heads"], m["dim"], m.get("vdim", m["dim"]),
                                                 m["decay_rank"], m["tau"], eps, dtype, linear_method, extra_out=width)
        else:
            raise ValueError(f"layer {index}: unknown mixer type {self.kind!r} (known: {_MIXERS})")
        self.norm1 = DynamicTanhNorm(width)
        mlp = layer.get("mlp")
        self.mlp = self.norm2 = None
        if mlp is not None:
            if mlp["kind"] != "dense":
                raise ValueError(f"layer {index}: unknown feed-forward kind {mlp['kind']!r}")
            self.mlp = PolyNormMLP(width, mlp["ff"], eps, dtype, linear_method)
            self.norm2 = DynamicTanhNorm(width)
        # weights of the embedding rows and of the outputs of layers 0 .. index in what the next layer reads
        self.depth_weights = nn.Parameter(torch.zeros(index + 2, dtype=torch.float32), requires_grad=False)
        self.depth_weights.data[-1] = 1.0

    def mixer(self, h: torch.Tensor, positions: torch.Tensor, cache: List[torch.Tensor], md: InputMetadata):
        """-> (the mixer's output, the pre-sigmoid gate on it), both [rows, width]."""
        if self.kind == "gla":
            return self.mix(h, cache, md)
        return self.mix(h, positions, cache, md)


class LalasunForCausalLM(nn.Module):
    uses_ragged_steps = True            # the runner lays every step out as a ragged batch
    supports_float32 = True

    def __init__(self, cfg: dict, dtype: torch.dtype, linear_method: Optional[LinearMethodBase] = None) -> None:
        super().__init__()
        if get_tensor_model_parallel_world_size() != 1:
            raise NotImplementedError("Lalasun layers keep a per-sequence state on one GPU: tensor parallelism is "
                                      "not built for them")
        if linear_method is not None:
            raise NotImplementedError("Lalasun checkpoints are dense: no quantised linear method")
        self.config, self.dtype = cfg, dtype
        self.mult = float(cfg.get("residual_mult", 1.0))
        self.embed_tokens = VocabParallelEmbedding(cfg["vocab"], cfg["width"], dtype)
        self.layers = nn.ModuleList([LalasunLayer(cfg, i, dtype, None) for i in range(len(cfg["layers"]))])
        self.norm = DynamicTanhNorm(cfg["width"])
        self.head = nn.Parameter(torch.zeros(cfg["vocab"], cfg["width"], dtype=dtype), requires_grad=False)
        self.sampler = Sampler(cfg["vocab"])
        self.register_buffer("unit_weight", torch.ones(1, dtype=torch.float32), persistent=False)
        # set by a caller that wants the stream after every layer (a debugging aid; costs a copy per layer)
        self.keep_residuals: Optional[list] = None

    # ------------------------------------------------------------------ caches
    @staticmethod
    def note_tensor_shapes(cfg: dict, shapes: Dict[str, tuple]) -> None:
        """The rank of a gla layer's low-rank decay projection is a tensor's shape, not a key of config.json."""
        for i, layer in enumerate(cfg["layers"]):
            name = f"l{i}.mix.a1"
            if layer["type"] == "gla" and name in shapes:
                layer["mixer"]["decay_rank"] = int(shapes[name][0])

    @staticmethod
    def cache_layout(cfg: dict, block_size: int) -> List[dict]:
        """Per layer: {"paged": [shape per page, ...]} for an attention layer (one tensor of latent rows, or keys and
        values), {"state": [shape per slot]} for a gla layer (state tensors are fp32, paged ones have the model's
        dtype)."""
        out = []
        for i, layer in enumerate(cfg["layers"]):
            m = layer["mixer"]
            if layer["type"] == "latent_attention":
                out.append({"paged": [(block_size, m["kv_rank"] + m["rot_dim"])]})
            elif layer["type"] == "attention":
                g = m.get("kv_heads", m["heads"])
                out.append({"paged": [(block_size, g * m["dim"]), (block_size, g * m.get("vdim", m["dim"]))]})
            elif layer["type"] == "gla":
                out.append({"state": [(m["heads"], m["dim"], m.get("vdim", m["dim"]))]})
            else:
                raise ValueError(f"layer {i}: unknown mixer type {layer['type']!r} (known: {_MIXERS})")
        return out

    # ----------------------------------------------------------------- forward
    def forward(self, input_ids, positions, kv_caches, input_metadata: InputMetadata):
        if input_metadata.ragged is None:
            raise RuntimeError("Lalasun steps need the ragged layout (InputMetadata.ragged)")
        positions = positions.reshape(-1)
        n = len(self.layers)
        x = self.embed_tokens(input_ids).float()
        # history[j]: X_j, the embedding rows and every layer's output before the depth mix; x: what the next layer reads.
        # The first launch files the embedding rows as entry 0 (a "mix" of that one entry) and takes the first norm.
        history = torch.empty(n + 1, x.shape[0], x.shape[1], dtype=torch.float32, device=x.device)
        h = (self.layers[0].norm1 if n else self.norm).gated_add_norm(x, self.dtype, history=history[:1],
                                                                      depth_weights=self.unit_weight)
        for i, layer in enumerate(self.layers):
            y, gate = layer.mixer(h, positions, kv_caches[i], input_metadata)
            if layer.mlp is not None:
                h = layer.norm2.gated_add_norm(x, self.dtype, y, gate, self.mult)
                y, gate = layer.mlp(h)
            nxt = self.layers[i + 1].norm1 if i + 1 < n else self.norm
            h = nxt.gated_add_norm(x, self.dtype, y, gate, self.mult, history[:i + 2], layer.depth_weights.data)
            if self.keep_residuals is not None:
                self.keep_residuals.append(x.clone())
        return h

    def sample(self, hidden_states, sampling_metadata: SamplingMetadata):
        return self.sampler(self.head, hidden_states, sampling_metadata)

    def compute_logits(self, hidden_rows: torch.Tensor) -> torch.Tensor:
        """fp32 logits of the given rows of ``forward``'s result: products accumulated and kept in fp32."""
        w = self.head
        out = torch.empty(hidden_rows.shape[0], w.shape[0], dtype=torch.float32, device=hidden_rows.device)
        rows32 = hidden_rows.float()
        step = 1 << 14                                        # bounds the fp32 copy of the matrix's slice
        for lo in range(0, w.shape[0], step):
            out[:, lo:lo + step] = torch.matmul(rows32, w[lo:lo + step].float().t())
        return out

    # ----------------------------------------------------------------- weights
    @torch.no_grad()
    def finish_random_init(self, seed: int) -> None:
        """After the loader's generic random values (no checkpoint): norms, activation numbers, decay biases and depth
        weights of a working model's size."""
        g = torch.Generator(device="cpu").manual_seed(seed)

        def rnd(shape, scale):
            return scale * torch.randn(shape, generator=g)

        def norm(nm: DynamicTanhNorm):
            nm.alpha.data.fill_(0.5)
            nm.weight.data.copy_(1.0 + rnd(nm.weight.shape, 0.1))
            nm.bias.data.copy_(rnd(nm.bias.shape, 0.02))
        for i, layer in enumerate(self.layers):
            norm(layer.norm1)
            if layer.mlp is not None:
                norm(layer.norm2)
                layer.mlp.act.coef.data.copy_(torch.tensor([1.0, 0.3, 0.1, 0.0]))
            if isinstance(layer.mix, GatedLinearAttentionMixer):
                layer.mix.out_norm.data.fill_(1.0)
                layer.mix.decay_bias.data.copy_(2.0 + rnd(layer.mix.decay_bias.shape, 1.0))
            if isinstance(layer.mix, LalasunLatentAttention):
                layer.mix.attn.latent_norm.data.fill_(1.0)
            w = torch.full((i + 2,), 0.1 / (i + 1))
            w[-1] = 0.9
            layer.depth_weights.data.copy_(w)
        norm(self.norm)

    def load_weights(self, state: Dict[str, torch.Tensor]) -> None:
        """``state``: checkpoint tensors by name ('embed', 'l<i>.mix.*', 'l<i>.mlp.*', 'l<i>.norm1[.alpha|.b]',
        'l<i>.rg1[.b]', 'l<i>.dwa', 'final.norm[.alpha|.b]', 'head')."""
        def cast(t):
            return t.to(self.dtype) if t.dtype.is_floating_point else t
        self.embed_tokens.weight.data.copy_(cast(state["embed"]))
        self.head.data.copy_(cast(state["head"]))
        self.norm.load_named(state, "final.norm")
        for i, layer in enumerate(self.layers):
            pre = f"l{i}."
            # norm parameters, decay biases, activation numbers and depth weights stay as stored: kept in fp32
            w = {k[len(pre) + 4:]: cast(v) for k, v in state.items() if k.startswith(pre + "mix.")}
            gate_w, gate_b = cast(state[pre + "rg1"]), cast(state[pre + "rg1.b"])
            if layer.kind == "gla":
                layer.mix.load_named(w, {"weight": gate_w, "bias": gate_b})
            else:
                layer.mix.load_named(w, gate_w, gate_b)
            layer.norm1.load_named(state, pre + "norm1")
            if layer.mlp is not None:
                layer.norm2.load_named(state, pre + "norm2")
                layer.mlp.load_named({k[len(pre) + 4:]: cast(v) for k, v in state.items() if k.startswith(pre + "mlp.")},
                                     cast(state[pre + "rg2"]), cast(state[pre + "rg2.b"]))
            layer.depth_weights.data.copy_(state[pre + "dwa"].float())

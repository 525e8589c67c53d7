"""Bogetar: a decoder whose layers are listed one by one in its config.json, with a norm before AND after every
sublayer, taken in groups of channels, and a short causal convolution added to what every sublayer reads.

Each entry of ``layers`` names the layer's token mixer -- ``delta`` (the delta rule with a gate and one decay per
head, behind short convolutions on q, k, v) or ``parallel`` (two mixers side by side on the same input: attention
over a sliding window whose weights are sigmoids of the biased scores instead of a softmax, with a per-head query /
key norm, rotary embedding on half-split pairs and a sigmoid output gate; and gated linear attention with a decay
per head and key channel; the two results are summed with the config's scales) -- with the mixer's sizes, and its
feed-forward: routed experts with a softmax router (``moe``) or none.

A layer, with N(u; w) the RMS norm in ``norm.groups`` groups of channels and C(u; c) = u + causal_conv(u; c):
    a = C(N(x; norm1); canon1);   x = x + ls1 * N(mixer(a); norm1b)
    b = C(N(x; norm2); canon2);   x = x + ls2 * N(ff(b); norm2b)
The stream x is fp32; the add of a sublayer's normed, scaled output and the norm that the next sublayer reads are
one kernel; the convolution's last inputs are per-sequence state like the recurrences' states.  The logits reuse
the embedding table.  Steps arrive in the ragged layout (``InputMetadata.ragged``): any mix of prompt portions and
decoded tokens.

Per layer the worker allocates what ``cache_layout`` asks for: pages of keys / values for a layer with attention,
per-sequence state slots for the convolutions' inputs and the recurrent states.
"""
from typing import Dict, List, Optional

import torch
import torch.nn as nn

from ..input_metadata import InputMetadata
from ..layers.attention import SigmoidWindowAttention
from ..layers.basic import CausalConvResidual, GroupRMSNorm, rotary_frequencies
from ..layers.linear import LinearMethodBase, MergedColumnParallelLinear, RowParallelLinear
from ..layers.moe import GroupRoutedExperts
from ..layers.recurrent import GatedDeltaMixer, GatedLinearAttentionMixer
from ..layers.sampler import Sampler, SamplingMetadata
from ..layers.vocab_parallel_embedding import VocabParallelEmbedding
from ..parallel_state import get_tensor_model_parallel_world_size

_MIXERS = ("delta", "parallel")


def normalize_config(raw: dict) -> dict:
    """The engine's generic geometry keys for a Bogetar config.json."""
    cfg = dict(raw)
    cfg["architecture"] = "bogetar"
    cfg["vocab_size"] = raw["vocab"]
    cfg["hidden_size"] = raw["width"]
    cfg["num_hidden_layers"] = len(raw["layers"])
    attn = [l["mixer"]["left"] for l in raw["layers"] if l["type"] == "parallel"]
    cfg["num_attention_heads"] = attn[0]["heads"] if attn else 1
    cfg["num_key_value_heads"] = attn[0].get("kv_heads", attn[0]["heads"]) if attn else 1
    cfg.setdefault("max_position_embeddings", 1 << 20)       # angles come from fp32 positions: no table to outgrow
    cfg.setdefault("torch_dtype", "bfloat16")
    return cfg


_DEFAULT_DECAY_RANK = 16          # of a model without a checkpoint whose config does not name one


def _decay_rank(right: dict) -> int:
    return int(right.get("decay_rank", _DEFAULT_DECAY_RANK))


def _left_sizes(m: dict):
    h, d = m["heads"], m["dim"]
    return h, m.get("kv_heads", h), d, m.get("vdim", d)


class ParallelMixer(nn.Module):
    """Sigmoid-weight window attention (``left``) and gated linear attention (``right``) on the same input: all
    projections of the input are ONE GEMM (left q | k | v | gate, right q | k | v | gate | first decay factor); each
    side has its output projection; the caller adds left_scale * left + right_scale * right."""

    def __init__(self, width: int, m: dict, eps: float, dtype, linear_method) -> None:
        super().__init__()
        left, right = m["left"], m["right"]
        h, g, d, dv = _left_sizes(left)
        rh, rd = right["heads"], right["dim"]
        rdv = right.get("vdim", rd)
        self.left_scale, self.right_scale = float(m.get("left_scale", 1.0)), float(m.get("right_scale", 1.0))
        self.sizes = [h * d, g * d, g * dv, h * dv, rh * rd, rh * rd, rh * rdv, rh * rdv, _decay_rank(right)]
        self.in_proj = MergedColumnParallelLinear(width, self.sizes, False, dtype, linear_method)
        rot = left.get("rot")
        freqs = rotary_frequencies(rot["dims"], rot["base"]) if rot else None
        window = (left.get("mask") or {}).get("size", 0)
        self.attn = SigmoidWindowAttention(h, g, d, dv, left["scale"], freqs, window, qk_norm_eps=eps, pair_halves=True)
        self.gla = GatedLinearAttentionMixer(width, rh, rd, rdv, _decay_rank(right), right["tau"], eps, dtype,
                                             linear_method, project=False)
        self.left_o = RowParallelLinear(h * dv, width, False, dtype, linear_method)
        self.right_o = RowParallelLinear(rh * rdv, width, False, dtype, linear_method)

    def state_shapes(self):
        return self.gla.state_shapes()

    def forward(self, a: torch.Tensor, positions: torch.Tensor, pages: List[torch.Tensor], state: torch.Tensor,
                md: InputMetadata):
        proj = self.in_proj(a)
        cols, lo = [], 0
        for n in self.sizes:
            cols.append(proj[:, lo:lo + n])
            lo += n
        left = self.attn(cols[0], cols[1], cols[2], cols[3], positions, pages[0], pages[1], md)
        right = self.gla.core(cols[4], cols[5], cols[6], cols[7], cols[8], state, md)
        return self.left_o(left), self.right_o(right)

    def load_named(self, w: Dict[str, torch.Tensor]) -> None:
        """``w``: left.{q, k, v, g, o, q.norm, k.norm, pb}, right.{q, k, v, g, a1, a2, a2.b, norm, o}."""
        self.in_proj.weight.data.copy_(torch.cat(
            [w["left.q"], w["left.k"], w["left.v"], w["left.g"], w["right.q"], w["right.k"], w["right.v"],
             w["right.g"], w["right.a1"]], 0))
        self.attn.q_norm.data.copy_(w["left.q.norm"].float())
        self.attn.k_norm.data.copy_(w["left.k.norm"].float())
        self.attn.score_bias.data.copy_(w["left.pb"].float())
        self.left_o.weight.data.copy_(w["left.o"])
        self.right_o.weight.data.copy_(w["right.o"])
        self.gla.load_named({k[6:]: v for k, v in w.items() if k.startswith("right.")})


def _experts(width: int, mlp: dict, dtype, index: int) -> GroupRoutedExperts:
    if mlp.get("kind") != "moe":
        raise ValueError(f"layer {index}: unknown feed-forward kind {mlp.get('kind')!r}")
    r, e = mlp["router"], mlp["expert"]
    groups = r.get("groups") or {"count": 1, "keep": 1}
    return GroupRoutedExperts(width, r["experts"], r["top"], e["ff"], None, groups["count"], groups["keep"], 1.0, dtype,
                              None, score="softmax", group_score="max", normalize=False, activation="clamped_glu",
                              limit=e.get("limit", float("inf")))


class BogetarLayer(nn.Module):
    def __init__(self, cfg: dict, index: int, dtype, linear_method) -> None:
        super().__init__()
        layer = cfg["layers"][index]
        width, eps, groups = cfg["width"], cfg["norm"]["eps"], cfg["norm"].get("groups", 1)
        taps, m = cfg["canon"]["taps"], layer["mixer"]
        self.kind = layer["type"]
        if self.kind == "delta":
            self.mix = GatedDeltaMixer(width, m["heads"], m.get("kv_heads", m["heads"]), m["dim"],
                                       m.get("vdim", m["dim"]), m["conv"], eps, dtype, linear_method)
        elif self.kind == "parallel":
            self.mix = ParallelMixer(width, m, eps, dtype, linear_method)
        else:
            raise ValueError(f"layer {index}: unknown mixer type {self.kind!r} (known: {_MIXERS})")
        self.norm1, self.norm1b = GroupRMSNorm(width, groups, eps), GroupRMSNorm(width, groups, eps)
        self.canon1 = CausalConvResidual(width, taps)
        self.ls1 = nn.Parameter(torch.ones(width, dtype=torch.float32), requires_grad=False)
        self.mlp = self.norm2 = self.norm2b = self.canon2 = self.ls2 = None
        if layer.get("mlp") is not None:
            self.mlp = _experts(width, layer["mlp"], dtype, index)
            self.norm2, self.norm2b = GroupRMSNorm(width, groups, eps), GroupRMSNorm(width, groups, eps)
            self.canon2 = CausalConvResidual(width, taps)
            self.ls2 = nn.Parameter(torch.ones(width, dtype=torch.float32), requires_grad=False)


class BogetarForCausalLM(nn.Module):
    uses_ragged_steps = True            # the runner lays every step out as a ragged batch
    supports_float32 = True

    def __init__(self, cfg: dict, dtype: torch.dtype, linear_method: Optional[LinearMethodBase] = None) -> None:
        super().__init__()
        if get_tensor_model_parallel_world_size() != 1:
            raise NotImplementedError("Bogetar layers keep a per-sequence state on one GPU: tensor parallelism is "
                                      "not built for them")
        if linear_method is not None:
            raise NotImplementedError("Bogetar checkpoints are dense: no quantised linear method")
        self.config, self.dtype = cfg, dtype
        self.embed_tokens = VocabParallelEmbedding(cfg["vocab"], cfg["width"], dtype)
        self.layers = nn.ModuleList([BogetarLayer(cfg, i, dtype, None) for i in range(len(cfg["layers"]))])
        self.norm = GroupRMSNorm(cfg["width"], cfg["norm"].get("groups", 1), cfg["norm"]["eps"])
        self.sampler = Sampler(cfg["vocab"])
        # set by a caller that wants the stream after every layer (a debugging aid; costs a copy per layer)
        self.keep_residuals: Optional[list] = None

    # ------------------------------------------------------------------ caches
    @staticmethod
    def note_tensor_shapes(cfg: dict, shapes: Dict[str, tuple]) -> None:
        """The rank of the gated linear attention's low-rank decay projection is a tensor's shape, not a key of
        config.json."""
        for i, layer in enumerate(cfg["layers"]):
            name = f"l{i}.mix.right.a1"
            if layer["type"] == "parallel" and name in shapes:
                layer["mixer"]["right"]["decay_rank"] = int(shapes[name][0])

    @staticmethod
    def cache_layout(cfg: dict, block_size: int) -> List[dict]:
        """Per layer {"paged": [...], "state": [...]}: pages of keys and values for a layer with attention; state
        slots (fp32) in this order: the last inputs of the convolution before the mixer, those of the one before the
        feed-forward (if the layer has one), then the mixer's own (delta: its convolutions' inputs and the rule's
        state; parallel: the linear attention's state)."""
        width, keep = cfg["width"], cfg["canon"]["taps"] - 1
        out = []
        for i, layer in enumerate(cfg["layers"]):
            m = layer["mixer"]
            state = [(keep, width)] * (2 if layer.get("mlp") is not None else 1)
            spec = {}
            if layer["type"] == "delta":
                h, g, d = m["heads"], m.get("kv_heads", m["heads"]), m["dim"]
                dv = m.get("vdim", d)
                state += [(m["conv"] - 1, 2 * g * d + h * dv), (h, d, dv)]
            elif layer["type"] == "parallel":
                h, g, d, dv = _left_sizes(m["left"])
                r = m["right"]
                spec["paged"] = [(block_size, g * d), (block_size, g * dv)]
                state += [(r["heads"], r["dim"], r.get("vdim", r["dim"]))]
            else:
                raise ValueError(f"layer {i}: unknown mixer type {layer['type']!r} (known: {_MIXERS})")
            spec["state"] = state
            out.append(spec)
        return out

    # ----------------------------------------------------------------- forward
    def forward(self, input_ids, positions, kv_caches, input_metadata: InputMetadata):
        if input_metadata.ragged is None:
            raise RuntimeError("Bogetar steps need the ragged layout (InputMetadata.ragged)")
        md = input_metadata
        positions = positions.reshape(-1)
        x = self.embed_tokens(input_ids).float()
        n = len(self.layers)
        if n == 0:
            return self.norm(x, self.dtype)
        h = self.layers[0].norm1(x, torch.float32)           # the convolution reads the norm unrounded
        for i, layer in enumerate(self.layers):
            cache = kv_caches[i]
            pages = cache[:2] if layer.kind == "parallel" else []
            state = cache[len(pages):]
            own = state[2 if layer.mlp is not None else 1:]
            a = layer.canon1(h, state[0], md, self.dtype)
            last = i + 1 == n
            nxt = layer.norm2 if layer.mlp is not None else (self.norm if last else self.layers[i + 1].norm1)
            out_dtype = self.dtype if (layer.mlp is None and last) else torch.float32
            if layer.kind == "parallel":
                left, right = layer.mix(a, positions, pages, own[0], md)
                h = layer.norm1b.add_norm(x, left, layer.ls1.data, nxt, out_dtype, right, layer.mix.left_scale,
                                          layer.mix.right_scale)
            else:
                h = layer.norm1b.add_norm(x, layer.mix(a, own, md), layer.ls1.data, nxt, out_dtype)
            if layer.mlp is not None:
                b = layer.canon2(h, state[1], md, self.dtype)
                _, y = layer.mlp(b)                            # fp32: the experts' weighted sum
                nxt = self.norm if last else self.layers[i + 1].norm1
                h = layer.norm2b.add_norm(x, y, layer.ls2.data, nxt, self.dtype if last else torch.float32)
            if self.keep_residuals is not None:
                self.keep_residuals.append(x.clone())
        return h

    def sample(self, hidden_states, sampling_metadata: SamplingMetadata):
        return self.sampler(self.embed_tokens.weight, hidden_states, sampling_metadata)

    def compute_logits(self, hidden_rows: torch.Tensor) -> torch.Tensor:
        """fp32 logits of the given rows of ``forward``'s result: products accumulated and kept in fp32."""
        w = self.embed_tokens.weight
        out = torch.empty(hidden_rows.shape[0], w.shape[0], dtype=torch.float32, device=hidden_rows.device)
        rows32 = hidden_rows.float()
        step = 1 << 14                                        # bounds the fp32 copy of the table's slice
        for lo in range(0, w.shape[0], step):
            out[:, lo:lo + step] = torch.matmul(rows32, w[lo:lo + step].float().t())
        return out

    # ----------------------------------------------------------------- weights
    @torch.no_grad()
    def finish_random_init(self, seed: int) -> None:
        """After the loader's generic random values (no checkpoint): norm weights, layer scales, convolution taps,
        decay biases and routers of a working model's size."""
        g = torch.Generator(device="cpu").manual_seed(seed)

        def rnd(t: torch.Tensor, scale: float, mean: float = 0.0) -> None:
            t.data.copy_(mean + scale * torch.randn(t.shape, generator=g))
        for layer in self.layers:
            for nm in (layer.norm1, layer.norm1b, layer.norm2, layer.norm2b):
                if nm is not None:
                    rnd(nm.weight, 0.1, 1.0)
            for canon in (layer.canon1, layer.canon2):
                if canon is not None:
                    rnd(canon.taps, 0.2)
            for ls in (layer.ls1, layer.ls2):
                if ls is not None:
                    rnd(ls, 0.05, 0.5)
            if isinstance(layer.mix, GatedDeltaMixer):
                rnd(layer.mix.conv_taps, 0.4)
                rnd(layer.mix.dt_bias, 0.5)
                rnd(layer.mix.a_log, 0.3)
                layer.mix.out_norm.data.fill_(1.0)
            else:
                layer.mix.gla.out_norm.data.fill_(1.0)
                rnd(layer.mix.gla.decay_bias, 1.0, 2.0)
                rnd(layer.mix.attn.score_bias, 0.5, -3.0)
                layer.mix.attn.q_norm.data.fill_(1.0)
                layer.mix.attn.k_norm.data.fill_(1.0)
            if layer.mlp is not None:
                rnd(layer.mlp.router, layer.mlp.width ** -0.5)
                layer.mlp.correction.data.zero_()
        rnd(self.norm.weight, 0.1, 1.0)

    def load_weights(self, state: Dict[str, torch.Tensor]) -> None:
        """``state``: checkpoint tensors by name ('embed', 'l<i>.mix.*', 'l<i>.mlp.*', 'l<i>.norm1[b]', 'l<i>.norm2[b]',
        'l<i>.ls1', 'l<i>.ls2', 'l<i>.canon1', 'l<i>.canon2', 'final.norm')."""
        def cast(t):
            return t.to(self.dtype) if t.dtype.is_floating_point else t
        self.embed_tokens.weight.data.copy_(cast(state["embed"]))
        self.norm.weight.data.copy_(state["final.norm"].float())
        for i, layer in enumerate(self.layers):
            pre = f"l{i}."
            # norm weights, layer scales, taps, biases and routers stay as stored: their layers keep them in fp32
            layer.mix.load_named({k[len(pre) + 4:]: cast(v) for k, v in state.items() if k.startswith(pre + "mix.")})
            for name in ("norm1", "norm1b", "norm2", "norm2b"):
                if getattr(layer, name) is not None:
                    getattr(layer, name).weight.data.copy_(state[pre + name].float())
            layer.ls1.data.copy_(state[pre + "ls1"].float())
            layer.canon1.taps.data.copy_(state[pre + "canon1"].float())
            if layer.mlp is not None:
                layer.ls2.data.copy_(state[pre + "ls2"].float())
                layer.canon2.taps.data.copy_(state[pre + "canon2"].float())
                layer.mlp.load_named({k[len(pre) + 4:]: (v if k.endswith("router") else cast(v))
                                      for k, v in state.items() if k.startswith(pre + "mlp.")})

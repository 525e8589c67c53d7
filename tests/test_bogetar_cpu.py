"""Bogetar without a GPU: configuration, cache layout and registry, and the plain statement's own mechanisms against
closed forms."""
import json
import os

import torch

import bogetar_util as bu
from oracle import bogetar as oracle

F64 = torch.float64


def _cfg():
    return bu.config([bu.parallel(4, 2, 16, 24, window=9, rot_dims=8), bu.delta(3, 1, 12, 8, conv=4), bu.delta(2, 2, 6, 10, conv=2)],
                     [bu.moe(6, 2, 20, 3, 2, 1.0), None, bu.moe(4, 1, 8, 1, 1, 0.5)], width=48, groups=4, taps=3)


def test_configuration_registry_and_cache_layout(tmp_path):
    from splitwise_amd.config import ModelConfig
    from splitwise_amd.model_executor.models.bogetar import BogetarForCausalLM
    cfg = _cfg()
    sd = bu.random_weights(cfg, 1, decay_rank=7)
    path = bu.write_model(str(tmp_path / "m"), cfg, sd)
    mc = ModelConfig(path, "float32")
    assert mc.architecture == "bogetar" and mc.uses_ragged_steps and mc.model_class() is BogetarForCausalLM
    assert mc.get_vocab_size() == cfg["vocab"] and mc.get_hidden_size() == cfg["width"]
    # a layer with attention holds pages AND state; the convolutions' last inputs come first among the state tensors
    assert mc.get_cache_layout(16) == [
        {"paged": [(16, 32), (16, 48)], "state": [(2, 48), (2, 48), (3, 10, 12)]},
        {"state": [(2, 48), (3, 2 * 12 + 3 * 8), (3, 12, 8)]},
        {"state": [(2, 48), (2, 48), (1, 2 * 12 + 2 * 10), (2, 6, 10)]}]
    from splitwise_amd.model_executor.model_loader import _safetensors_shapes
    BogetarForCausalLM.note_tensor_shapes(mc.hf_config, _safetensors_shapes(os.path.join(path, "model.safetensors")))
    assert mc.hf_config["layers"][0]["mixer"]["right"]["decay_rank"] == 7
    with open(os.path.join(path, "config.json")) as f:
        assert json.load(f)["architecture"] == "Bogetar"


def test_layered_cache_holds_pages_and_state_of_one_layer():
    from splitwise_amd.worker.cache_engine import LayeredCacheEngine
    layout = [{"paged": [(16, 32), (16, 48)], "state": [(2, 48), (3, 10, 12)]}, {"state": [(1, 8)]}, {"paged": [(16, 4)]}]
    cache = LayeredCacheEngine.allocate(layout, 5, 3, torch.bfloat16, torch.device("cpu"))
    assert [tuple(t.shape) for t in cache[0]] == [(5, 16, 32), (5, 16, 48), (3, 2, 48), (3, 3, 10, 12)]
    assert [t.dtype for t in cache[0]] == [torch.bfloat16, torch.bfloat16, torch.float32, torch.float32]
    assert [tuple(t.shape) for t in cache[1]] == [(3, 1, 8)] and [tuple(t.shape) for t in cache[2]] == [(5, 16, 4)]


def test_bench_presets_are_whole_models():
    from splitwise_amd.config import ModelConfig
    for name in ("bogetar-2k", "bogetar-4k"):
        mc = ModelConfig(name, "bfloat16")
        layout = mc.get_cache_layout(16)
        assert len(layout) == len(mc.hf_config["layers"]) == 10
        assert any("paged" in spec for spec in layout) and all("state" in spec for spec in layout)


def test_group_norm_and_convolution_against_closed_forms():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(5, 24, generator=g, dtype=F64)
    w = torch.randn(24, generator=g, dtype=F64)
    out = oracle.group_norm(x, w, 3, 0.0)
    assert torch.allclose((out / w).view(5, 3, 8).pow(2).mean(-1), torch.ones(5, 3, dtype=F64))     # every group has unit mean square
    assert torch.allclose(oracle.group_norm(x, w, 1, 1e-5), x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + 1e-5) * w)
    taps = torch.randn(24, 3, generator=g, dtype=F64)
    y = oracle.causal_conv(x, taps)
    assert torch.allclose(y[0], taps[:, 2] * x[0]) and torch.allclose(y[1], taps[:, 2] * x[1] + taps[:, 1] * x[0])
    assert torch.allclose(y[4], taps[:, 2] * x[4] + taps[:, 1] * x[3] + taps[:, 0] * x[2])


def test_sigmoid_weights_window_and_bias():
    g = torch.Generator().manual_seed(1)
    n, H, G, d, dv = 19, 4, 2, 6, 5
    q, k, v = (torch.randn(n, h, s, generator=g, dtype=F64) for h, s in ((H, d), (G, d), (G, dv)))
    bias = torch.tensor([-1.0, 0.0, 0.5, 2.0], dtype=F64)
    ones = torch.ones(n, G, 1, dtype=F64)
    total = oracle.sigmoid_window_attention(q, k, ones, bias, 0.4, 5)[..., 0]                       # sums of the weights
    t, a = n - 1, 3
    assert torch.allclose(total[t, a], torch.sigmoid((k[t - 4:t + 1, a // 2] @ q[t, a]) * 0.4 + 2.0).sum())
    assert total.max() > 1.5                                                                        # not normalised
    # a key one past the window changes nothing, the window's last one does
    for j, seen in ((t - 5, False), (t - 4, True)):
        k2 = k.clone()
        k2[j] += 3.0
        changed = (oracle.sigmoid_window_attention(q, k2, v, bias, 0.4, 5)[t] - oracle.sigmoid_window_attention(q, k, v, bias, 0.4, 5)[t])
        assert (changed.abs().max() > 1e-6) == seen
    # a window of one: every position sees itself only
    own = oracle.sigmoid_window_attention(q, k, v, bias, 0.4, 1)
    assert torch.allclose(own[7, 1], torch.sigmoid((k[7, 0] @ q[7, 1]) * 0.4 + 0.0) * v[7, 0])


def test_delta_rule_overwrites_a_key_and_forgets_with_its_decay():
    """With beta = 1 and decay = 1 a unit key's value is replaced by the new one; a decay g scales what was there."""
    d, dv = 4, 3
    e0 = torch.eye(d, dtype=F64)[0]
    k = e0.view(1, 1, d).repeat(2, 1, 1)
    v = torch.tensor([[[1.0, 2.0, 3.0]], [[-4.0, 0.5, 9.0]]], dtype=F64)
    one = torch.ones(2, 1, dtype=F64)
    o, S = oracle.gated_delta_scan(k, k, v, one, one)
    assert torch.allclose(o[:, 0], v[:, 0]) and torch.allclose(S[0, 0], v[1, 0])
    o, S = oracle.gated_delta_scan(k, k, v, 0.5 * one, torch.tensor([[1.0], [0.25]], dtype=F64))
    # after token 0: S = 0.5 v0;  token 1: S <- 0.25 * 0.5 v0, u = 0.5 (v1 - S), S += u
    want = 0.125 * v[0, 0] + 0.5 * (v[1, 0] - 0.125 * v[0, 0])
    assert torch.allclose(S[0, 0], want) and torch.allclose(o[1, 0], want)
    # the state carried from one call into the next equals one long run
    g = torch.Generator().manual_seed(2)
    q, kk = torch.randn(9, 2, d, generator=g, dtype=F64), oracle.unit(torch.randn(9, 2, d, generator=g, dtype=F64))
    vv, b, dec = torch.randn(9, 2, dv, generator=g, dtype=F64), torch.rand(9, 2, generator=g, dtype=F64), torch.rand(9, 2, generator=g, dtype=F64)
    whole, _ = oracle.gated_delta_scan(q, kk, vv, b, dec)
    first, S = oracle.gated_delta_scan(q[:4], kk[:4], vv[:4], b[:4], dec[:4])
    rest, _ = oracle.gated_delta_scan(q[4:], kk[4:], vv[4:], b[4:], dec[4:], S)
    assert torch.allclose(torch.cat([first, rest]), whole)


def test_router_keeps_the_best_groups_and_does_not_renormalise():
    z = torch.tensor([0.1, 0.2, 3.0, -1.0, 2.5, 2.4, 0.0, 0.3], dtype=F64)
    s = torch.softmax(z, -1)
    # four groups of two score 0.2, 3.0, 2.5, 0.3 (as logits): keep 2 -> groups 1 and 2; top 3 of experts 2, 3, 4, 5
    ids, w = oracle.route(z, 3, 4, 2)
    assert sorted(ids.tolist()) == [2, 4, 5] and torch.allclose(w.sum(), s[[2, 4, 5]].sum()) and w.sum() < 1
    # keep 1: only group 1 (experts 2 and 3), although expert 4 scores more than expert 3
    ids, _ = oracle.route(z, 2, 4, 1)
    assert sorted(ids.tolist()) == [2, 3]
    ids, w = oracle.route(z, 8, 1, 1)
    assert sorted(ids.tolist()) == list(range(8)) and torch.allclose(w.sum(), torch.tensor(1.0, dtype=F64))


def test_expert_limits():
    h = torch.tensor([1.0, -2.0], dtype=F64)
    gate, up = torch.tensor([[3.0, 0.0], [0.0, 1.0]], dtype=F64), torch.tensor([[0.0, 2.0], [5.0, 0.0]], dtype=F64)
    down = torch.eye(2, dtype=F64)
    # gate x = (3, -2) -> min(., 1) = (1, -2): no lower limit on the gate;  up x = (-4, 5) -> (-1, 1)
    out = oracle.expert(h, gate, up, down, 1.0)
    g = torch.tensor([1.0, -2.0], dtype=F64)
    assert torch.allclose(out, g * torch.sigmoid(1.702 * g) * torch.tensor([0.0, 2.0], dtype=F64))

"""Lalasun without a GPU: configuration, cache layout and registry, and the plain statement's own mechanisms against
closed forms."""
import json
import os

import torch

import lalasun_util as lu
from oracle import lalasun as oracle


def _cfg():
    return lu.config([lu.gla(2, 12, 20, 4.0), lu.latent(3, 8, 4, 12, 20, window=9), lu.attention(4, 2, 16, 8, chunk=11, rot_dims=8)],
                     [lu.dense(40), None, lu.dense(24)])


def test_configuration_registry_and_cache_layout(tmp_path):
    from splitwise_amd.config import ModelConfig
    from splitwise_amd.model_executor.models.lalasun import LalasunForCausalLM
    cfg = _cfg()
    sd = lu.random_weights(cfg, 1, decay_rank=7)
    path = lu.write_model(str(tmp_path / "m"), cfg, sd)
    mc = ModelConfig(path, "float32")
    assert mc.architecture == "lalasun" and mc.uses_ragged_steps and mc.model_class() is LalasunForCausalLM
    assert mc.get_vocab_size() == cfg["vocab"] and mc.get_hidden_size() == cfg["width"]
    assert mc.get_cache_layout(16) == [{"state": [(2, 12, 20)]}, {"paged": [(16, 24)]}, {"paged": [(16, 32), (16, 16)]}]
    # the rank of the decay projection is a tensor's shape
    from splitwise_amd.model_executor.model_loader import _safetensors_shapes
    LalasunForCausalLM.note_tensor_shapes(mc.hf_config, _safetensors_shapes(os.path.join(path, "model.safetensors")))
    assert mc.hf_config["layers"][0]["mixer"]["decay_rank"] == 7
    with open(os.path.join(path, "config.json")) as f:
        assert json.load(f)["architecture"] == "Lalasun"


def test_bench_presets_are_whole_models():
    from splitwise_amd.config import ModelConfig
    for name in ("lalasun-2k", "lalasun-4k"):
        mc = ModelConfig(name, "bfloat16")
        layout = mc.get_cache_layout(16)
        assert len(layout) == len(mc.hf_config["layers"]) == 10
        assert {next(iter(spec)) for spec in layout} == {"paged", "state"}


def test_masks_and_the_extra_softmax_term():
    g = torch.Generator().manual_seed(0)
    n, H, G, d, dv = 23, 4, 2, 6, 5
    q, k, v = (torch.randn(n, h, s, generator=g, dtype=torch.float64) for h, s in ((H, d), (G, d), (G, dv)))
    ones = torch.ones(n, G, 1, dtype=torch.float64)
    for window, chunk in ((0, 0), (5, 0), (0, 7), (1, 0), (0, 1)):
        total = oracle.masked_attention(q, k, ones, 0.4, window=window, chunk=chunk)           # sums of the weights
        assert torch.allclose(total, torch.ones_like(total))
        with_sink = oracle.masked_attention(q, k, ones, 0.4, window=window, chunk=chunk, sink=True)
        assert (with_sink < 1).all() and (with_sink > 0).all()
        # weight sum s / (1 + s) with s the sum of exp(score) over the visible keys
        t, a = n - 1, H - 1
        lo = max(0, t - window + 1) if window else (t // chunk) * chunk if chunk else 0
        s = torch.exp((k[lo:t + 1, a // (H // G)] @ q[t, a]) * 0.4).sum()
        assert torch.allclose(with_sink[t, a, 0], s / (1 + s))
    # a key outside the window / in the chunk before changes nothing
    k2, v2 = k.clone(), v.clone()
    k2[n - 1 - 5], v2[n - 1 - 5] = 50.0, -7.0
    a = oracle.masked_attention(q, k, v, 0.4, window=5)[n - 1]
    b = oracle.masked_attention(q, k2, v2, 0.4, window=5)[n - 1]
    assert torch.equal(a, b)
    k2, v2 = k.clone(), v.clone()
    k2[20], v2[20] = 50.0, -7.0                                        # position 20 ends the chunk [14, 21)
    assert torch.equal(oracle.masked_attention(q, k, v, 0.4, chunk=7)[21], oracle.masked_attention(q, k2, v2, 0.4, chunk=7)[21])
    assert not torch.equal(oracle.masked_attention(q, k, v, 0.4, chunk=7)[20], oracle.masked_attention(q, k2, v2, 0.4, chunk=7)[20])


def test_state_scan_against_its_unrolled_sum():
    g = torch.Generator().manual_seed(1)
    n, H, d, dv = 9, 2, 4, 3
    q, k = torch.randn(n, H, d, generator=g, dtype=torch.float64), torch.randn(n, H, d, generator=g, dtype=torch.float64)
    v = torch.randn(n, H, dv, generator=g, dtype=torch.float64)
    decay = oracle.channel_decay(torch.randn(n, H, d, generator=g, dtype=torch.float64) * 2, 3.0)
    assert (decay > 0).all() and (decay < 1).all()
    o, S = oracle.decayed_state_scan(q, k, v, decay)
    # o_t = sum_{j <= t} (q_t * prod_{j < s <= t} decay_s) . k_j  v_j
    for t in (0, 4, n - 1):
        want = torch.zeros(H, dv, dtype=torch.float64)
        for j in range(t + 1):
            keep = torch.ones(H, d, dtype=torch.float64)
            for s in range(j + 1, t + 1):
                keep = keep * decay[s]
            want += ((q[t] * keep * k[j]).sum(-1, keepdim=True)) * v[j]
        assert torch.allclose(o[t], want)
    # carried state: two halves equal the whole
    o1, S1 = oracle.decayed_state_scan(q[:5], k[:5], v[:5], decay[:5])
    o2, S2 = oracle.decayed_state_scan(q[5:], k[5:], v[5:], decay[5:], state=S1)
    assert torch.allclose(torch.cat([o1, o2]), o) and torch.allclose(S2, S)


def test_poly_norm_and_tanh_norm_closed_forms():
    z = torch.tensor([[1.0, -2.0, 3.0, 0.5]], dtype=torch.float64)
    c = torch.tensor([0.5, -1.0, 2.0, 0.25], dtype=torch.float64)
    rms = lambda u: torch.sqrt((u * u).mean() + 1e-5)                 # noqa: E731
    want = c[0] * z / rms(z) + c[1] * z ** 2 / rms(z ** 2) + c[2] * z ** 3 / rms(z ** 3) + c[3]
    assert torch.allclose(oracle.poly_norm(z, c, 1e-5), want)
    u = torch.tensor([0.3, -4.0], dtype=torch.float64)
    out = oracle.tanh_norm(u, torch.tensor(0.5), torch.tensor([2.0, 3.0]), torch.tensor([0.1, -0.1]))
    assert torch.allclose(out, torch.tanh(0.5 * u) * torch.tensor([2.0, 3.0]) + torch.tensor([0.1, -0.1]))

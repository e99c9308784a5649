"""Gezozen without a GPU: configuration round trip, tensor inventory, the library's rotation table against the oracle's, and the
oracle's mechanisms on hand-made inputs whose results are known by construction."""
import ctypes as C
import math

import pytest
import torch

from tests import gezozen_oracle as orc

F = torch.float64


def _spec():
    from vllm_rust_amd.gezozen import GezozenLayerSpec, GezozenSpec, RotationSpec
    stretch = {"factor": 8.0, "original": 64.0, "fast": 16.0, "slow": 2.0}
    layers = [GezozenLayerSpec(mixer="delta", heads=4, kv_heads=2, dim=6, vdim=10, conv=3, mlp="moe", experts=5, top=2, expert_ff=12, shared_ff=20),
              GezozenLayerSpec(mixer="parallel", heads=6, kv_heads=3, dim=8, vdim=4, scale=0.3, softcap=9.0, rot=RotationSpec(4, 100.0), r_heads=3,
                               r_dim=10, r_vdim=6, tau=4.0, decay_rank=7, left_scale=0.7, right_scale=1.3, mlp=None),
              GezozenLayerSpec(mixer="parallel_2", heads=2, kv_heads=1, dim=12, vdim=12, window=5, scale=0.25, rot=RotationSpec(8, 500.0, stretch),
                               r_heads=2, r_dim=6, r_vdim=14, decay=(0.9, 0.99), r_rot=RotationSpec(6, 1000.0), left_scale=1.1, right_scale=0.5,
                               mlp="moe", experts=3, top=1, expert_ff=9, shared_ff=0)]
    return GezozenSpec(vocab=37, width=24, layers=layers, norm_eps=1e-5, norm_groups=3, postln_alpha=2.5)


def test_config_round_trip():
    from vllm_rust_amd.gezozen import GezozenSpec
    spec = _spec()
    cfg = spec.to_config()
    assert cfg["architecture"] == "Gezozen" and [e["type"] for e in cfg["layers"]] == ["delta", "parallel", "parallel_2"]
    assert cfg["layers"][1]["mlp"] is None and "shared" not in cfg["layers"][2]["mlp"] and cfg["layers"][2]["mixer"]["left"]["mask"] == {"size": 5}
    assert "softcap" not in cfg["layers"][2]["mixer"]["left"] and "mask" not in cfg["layers"][1]["mixer"]["left"]
    # the decay projection's inner size is a shape of the checkpoint, not configuration
    assert GezozenSpec.from_config(cfg, {1: 7}) == spec
    assert GezozenSpec.from_config(cfg) != spec


def test_tensor_inventory_registry_and_oracle_runs():
    from vllm_rust_amd.gezozen import synthetic_weights
    from vllm_rust_amd.models import REGISTRY
    spec = _spec()
    shapes = spec.tensor_shapes()
    assert shapes["l0.mix.q"] == (12, 24) and shapes["l0.mix.v.conv"] == (40, 3) and shapes["l0.mix.a"] == (4, 24) and shapes["l0.mix.dt_bias"] == (4,)
    assert shapes["l0.mlp.shared.sg"] == (1, 24) and shapes["l0.mlp.e4.down"] == (24, 12) and "l0.mlp.e5.up" not in shapes
    assert shapes["l1.mix.left.q.norm"] == (8,) and shapes["l1.mix.right.a2"] == (30, 7) and shapes["l1.mix.right.norm"] == (6,)
    assert "l1.norm2" not in shapes and "l1.rg2" not in shapes and "l1.mix.left.q.b" not in shapes
    assert shapes["l2.mix.left.k.b"] == (12,) and "l2.mix.right.norm" not in shapes and "l2.mlp.shared.up" not in shapes
    ck = synthetic_weights(spec, 0)
    assert set(ck) == set(shapes) and all(tuple(ck[k].shape) == shapes[k] and ck[k].dtype == torch.bfloat16 for k in ck)
    assert "Gezozen" in REGISTRY
    lg, tr = orc.forward(spec.to_config(), {k: v.double() for k, v in ck.items()}, [3, 1, 4, 1, 5, 9, 2, 6, 5, 3])
    assert lg.shape == (10, 37) and tr.shape == (3, 10, 24) and bool(torch.isfinite(lg).all())
    # after a layer every norm group of the stream has the root mean square of its gains
    g = tr[0].reshape(10, 3, 8)
    w = ck["l0.norm2"].double().reshape(3, 8)
    assert float(((g / w).pow(2).mean(-1) - 1).abs().max()) < 1e-3


def test_library_rotation_table_matches_the_oracle():
    from vllm_rust_amd._lib import Rotation, lib
    cases = [dict(dims=8, base=500.0), dict(dims=24, base=2e4, scaling=dict(factor=8.0, original=1024, fast=16.0, slow=2.0)),
             dict(dims=64, base=1e6, scaling=dict(factor=16.0, original=512, fast=8.0, slow=0.5)),
             dict(dims=6, base=100.0, scaling=dict(factor=2.0, original=16, fast=4.0, slow=2.0)),
             dict(dims=16, base=1e4, scaling=dict(factor=3.0, original=4096, fast=1.0, slow=1.0))]
    for rot in cases:
        sc = rot.get("scaling") or {}
        r = Rotation(rot["dims"], rot["base"], sc.get("factor", 0.0), sc.get("original", 0.0), sc.get("fast", 0.0), sc.get("slow", 0.0))
        steps = (C.c_float * (rot["dims"] // 2))()
        mul = C.c_float()
        assert lib.vmx_rotation_steps(C.byref(r), steps, C.byref(mul)) == 0
        want, wmul = orc.rotation_steps(rot)
        assert abs(mul.value - wmul) < 1e-6
        for got, w in zip(steps, want):
            assert abs(got - w) <= 1e-6 * abs(w)
    # stretched: the first pair keeps its step, the last turns `factor` times slower, and the ramp between is monotone
    plain, _ = orc.rotation_steps(dict(dims=24, base=2e4))
    st, m = orc.rotation_steps(cases[1])
    assert st[0] == plain[0] and abs(st[-1] - plain[-1] / 8.0) < 1e-15 and m == pytest.approx(0.1 * math.log(8.0) + 1)
    ratio = [a / b for a, b in zip(st, plain)]
    assert all(x >= y - 1e-12 for x, y in zip(ratio, ratio[1:]))
    bad = Rotation(7, 100.0, 0, 0, 0, 0)
    assert lib.vmx_rotation_steps(C.byref(bad), steps, C.byref(mul)) != 0


def test_oracle_group_norm_and_rotation_in_halves():
    x = torch.tensor([[3.0, 4.0, 0.0, 0.0, 1.0, 1.0, 1.0, 1.0]], dtype=F)
    y = orc.group_rms_norm(x, torch.ones(8, dtype=F), 2, 0.0)
    assert torch.allclose(y[0, :4], x[0, :4] / 2.5) and torch.allclose(y[0, 4:], torch.ones(4, dtype=F))
    assert torch.allclose(orc.group_rms_norm(x, torch.ones(8, dtype=F), 1, 0.0), x / math.sqrt(x.pow(2).mean()))
    # coordinate 0 pairs with coordinate 2 (dims 4), coordinates 4, 5 pass
    rot = dict(dims=4, base=10.0)
    v = torch.tensor([[1.0, 0.0, 0.0, 0.0, 7.0, 8.0]], dtype=F)
    r = orc.rotate_halves(v, 3, rot)
    assert torch.allclose(r[0], torch.tensor([math.cos(3.0), 0.0, math.sin(3.0), 0.0, 7.0, 8.0], dtype=F))
    v = torch.tensor([[0.0, 1.0, 0.0, 0.0, 7.0, 8.0]], dtype=F)
    a = 3 * 10.0 ** -0.5
    assert torch.allclose(orc.rotate_halves(v, 3, rot)[0], torch.tensor([0.0, math.cos(a), 0.0, math.sin(a), 7.0, 8.0], dtype=F))
    # rotations keep q . k a function of the distance
    g = torch.Generator().manual_seed(0)
    q, k = torch.randn(1, 6, generator=g, dtype=F), torch.randn(1, 6, generator=g, dtype=F)
    d1 = (orc.rotate_halves(q, 9, rot) * orc.rotate_halves(k, 4, rot)).sum()
    d2 = (orc.rotate_halves(q, 105, rot) * orc.rotate_halves(k, 100, rot)).sum()
    assert abs(float(d1 - d2)) < 1e-9


def test_oracle_attention_window_and_soft_cap():
    T, D = 12, 4
    q, k = torch.zeros(T, 2, D, dtype=F), torch.zeros(T, 1, D, dtype=F)
    v = torch.arange(T, dtype=F).reshape(T, 1, 1).expand(T, 1, 3).clone()
    k[2, 0, 0] = 50.0
    q[:, :, 0] = 1.0
    o = orc.softmax_attention(q, k, v, 1.0, None, 5)
    assert float((o[6, 0] - 2.0).abs().max()) < 1e-9            # distance 4 < 5: key 2 decides
    assert float((o[7, 1] - 5.0).abs().max()) < 1e-9            # distance 5: gone; equal scores over 3 .. 7
    o = orc.softmax_attention(q, k, v, 1.0, None, None)
    assert float((o[11, 0] - 2.0).abs().max()) < 1e-9           # causal: visible from anywhere later
    o = orc.softmax_attention(q, k, v, 1.0, 2.0, None)          # capped at 2: key 2 weighs e^2 against ones
    w = math.exp(2.0) / (math.exp(2.0) + 3)
    assert float((o[3, 0] - (w * 2 + (1 - w) * (0 + 1 + 3) / 3)).abs().max()) < 1e-6


def test_oracle_matrix_memories():
    g = torch.Generator().manual_seed(1)
    T, H, D, V = 7, 2, 3, 4
    q, k, v = (torch.randn(T, H, n, generator=g, dtype=F) for n in (D, D, V))
    decay = torch.rand(T, H, D, generator=g, dtype=F)
    o = orc.decayed_outer_memory(q, k, v, decay)
    for t in (0, 3, 6):                                           # o_t = sum_j sum_d q_td (prod_{j < s <= t} decay_sd) k_jd v_j
        want = torch.zeros(H, V, dtype=F)
        for j in range(t + 1):
            w = decay[j + 1:t + 1].prod(0) if j < t else torch.ones(H, D, dtype=F)
            want += ((q[t] * w * k[j]).sum(-1, keepdim=True)) * v[j]
        assert torch.allclose(o[t], want, atol=1e-12)
    # delta rule: orthonormal keys, beta 1, no decay: every key reads back its own value, and a rewrite replaces it
    k = torch.eye(3, dtype=F).reshape(3, 1, 3).repeat(2, 1, 1)   # keys e0 e1 e2 e0 e1 e2
    v = torch.randn(6, 1, V, generator=g, dtype=F)
    ones = torch.ones(6, 1, dtype=F)
    o = orc.delta_rule_memory(k, k, v, ones, ones)
    assert torch.allclose(o, v, atol=1e-12)
    o = orc.delta_rule_memory(k[[0, 0, 0, 0, 0, 0]], k, v, ones, ones)      # always asking for e0
    assert torch.allclose(o[2], v[0], atol=1e-12) and torch.allclose(o[5], v[3], atol=1e-12)
    o = orc.delta_rule_memory(k[[0, 0, 0, 0, 0, 0]], k, v, 0.5 * ones, 0.0 * ones + torch.tensor([[1.0], [0], [0], [0], [0], [0]], dtype=F))
    assert torch.allclose(o[4], v[0] * 0.5 ** 4, atol=1e-12)      # written once, then only decays (the write's own step decays nothing)


def test_oracle_router_and_scaled_expert_input():
    W, E = 6, 4
    g = torch.Generator().manual_seed(2)
    w = {"r.router": torch.zeros(E, W, dtype=F)}
    w["r.router"][1, 0], w["r.router"][3, 0], w["r.router"][2, 0] = 2.0, 2.0, -1.0
    h = torch.zeros(2, W, dtype=F)
    h[0, 0], h[1, 0] = 1.0, -1.0
    ids, s = orc.route(h, w, "r.", 2)
    assert ids.tolist() == [[1, 3], [2, 0]]                       # a tie goes to the smaller index
    assert torch.allclose(s[0], torch.sigmoid(torch.tensor([2.0, 2.0], dtype=F))) and float(s[1, 1]) == 0.5
    for e in range(E):
        for n, shape in (("gate", (5, W)), ("up", (5, W)), ("down", (W, 5))):
            w[f"r.e{e}.{n}"] = torch.randn(shape, generator=g, dtype=F)
    out = orc.feed_forward(h, w, "r.", {"kind": "moe", "router": {"experts": E, "top": 2}, "expert": {"ff": 5}})
    want = sum(orc.glu_expert(s[0, j] * h[:1], w, f"r.e{e}.") for j, e in enumerate((1, 3)))
    assert torch.allclose(out[:1], want, atol=1e-12)
    # the weight inside the expert is not the weight outside it
    assert not torch.allclose(out[:1], sum(s[0, j] * orc.glu_expert(h[:1], w, f"r.e{e}.") for j, e in enumerate((1, 3))), atol=1e-6)
    w["r.shared.gate"], w["r.shared.up"], w["r.shared.down"] = (torch.randn(sh, generator=g, dtype=F) for sh in ((7, W), (7, W), (W, 7)))
    w["r.shared.sg"] = torch.randn(1, W, generator=g, dtype=F)
    out2 = orc.feed_forward(h, w, "r.", {"kind": "moe", "router": {"experts": E, "top": 2}, "expert": {"ff": 5}, "shared": {"ff": 7}})
    assert torch.allclose(out2 - out, orc.glu_expert(h, w, "r.shared.") * torch.sigmoid(h @ w["r.shared.sg"].T), atol=1e-12)


def test_oracle_short_convolution_order():
    x = torch.tensor([[1.0], [10.0], [100.0], [1000.0]], dtype=F)
    taps = torch.tensor([[3.0, 2.0, 1.0]], dtype=F)               # the last column meets the current token
    assert orc.short_conv(x, taps).reshape(-1).tolist() == [1.0, 12.0, 123.0, 1230.0]

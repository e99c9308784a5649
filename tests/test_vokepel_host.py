"""Vokepel without a GPU: configuration round trip, running order of looped layers, tensor inventory, and the oracle's mechanisms
on hand-made inputs whose results are known by construction."""
import math

import pytest
import torch

from tests import vokepel_oracle as orc

F = torch.float64


def _spec():
    from vllm_rust_amd.vokepel import VokepelLayerSpec, VokepelSpec
    layers = [VokepelLayerSpec(mixer="parallel", heads=4, kv_heads=2, dim=8, vdim=6, window=5, scale=0.3, rot_dims=4, rot_base=100.0, gru_width=12,
                               left_scale=0.7, right_scale=0.4, mlp="dense", ff=20),
              VokepelLayerSpec(mixer="attention", heads=6, kv_heads=3, dim=4, vdim=4, window=0, scale=0.5, softcap=7.0, mlp=None),
              VokepelLayerSpec(mixer="attention", heads=2, kv_heads=1, dim=6, vdim=6, window=3, scale=0.5, mlp="dense", ff=9)]
    return VokepelSpec(vocab=31, width=16, layers=layers, norm_eps=1e-5, residual_mult=0.5, logit_scale=0.8, logit_softcap=9.0, loop=(1, 3, 2))


def test_config_round_trip_and_running_order():
    from vllm_rust_amd.vokepel import VokepelSpec
    spec = _spec()
    cfg = spec.to_config()
    assert cfg["architecture"] == "Vokepel" and cfg["layers"][0]["type"] == "parallel" and cfg["layers"][1]["mlp"] is None
    assert VokepelSpec.from_config(cfg) == spec
    assert spec.layer_runs == [(0, None), (1, 0), (2, 0), (1, 1), (2, 1)] == orc.layer_runs(cfg)
    import dataclasses
    flat = dataclasses.replace(spec, loop=None, logit_softcap=0.0)
    assert "loop" not in flat.to_config() and VokepelSpec.from_config(flat.to_config()) == flat
    assert flat.layer_runs == [(0, None), (1, None), (2, None)]


def test_tensor_inventory_and_registry():
    from vllm_rust_amd.models import REGISTRY
    from vllm_rust_amd.vokepel import synthetic_weights
    spec = _spec()
    shapes = spec.tensor_shapes()
    assert shapes["loop.in"] == (16, 32) and shapes["loop.step"] == (2, 16)
    assert shapes["l0.mix.left.v"] == (12, 16) and shapes["l0.mix.right.o"] == (16, 12) and shapes["l0.mix.left.sink"] == (4,)
    assert shapes["l1.mix.talk"] == (6, 6) and shapes["l1.mix.k.norm"] == (12,) and "l1.norm2" not in shapes and "l1.mix.v" not in shapes
    ck = synthetic_weights(spec, 0)
    assert set(ck) == set(shapes) and all(tuple(ck[k].shape) == shapes[k] and ck[k].dtype == torch.bfloat16 for k in ck)
    assert "Vokepel" in REGISTRY
    lg, tr = orc.forward(spec.to_config(), {k: v.double() for k, v in ck.items()}, [3, 1, 4, 1, 5, 9, 2, 6])
    assert lg.shape == (8, 31) and tr.shape == (5, 8, 16) and bool(torch.isfinite(lg).all()) and float(lg.abs().max()) <= 9.0


def test_oracle_window_sink_and_distance_penalty():
    T, D = 6, 4
    q = torch.zeros(T, 1, D, dtype=F)          # all scores 0: uniform weights over what is visible
    k = torch.randn(T, 1, D, dtype=F)
    v = torch.arange(T, dtype=F).reshape(T, 1, 1).repeat(1, 1, 2)
    out = orc.windowed_attention(q, k, v, 1.0, size=3)
    assert torch.allclose(out[:, 0, 0], torch.tensor([0.0, 0.5, 1.0, 2.0, 3.0, 4.0], dtype=F))      # means of the last <= 3 values
    out = orc.windowed_attention(q, k, v, 1.0, size=1)
    assert torch.allclose(out[:, 0, 0], torch.arange(T, dtype=F))
    # a sink of 0 is one more unit in the denominator: row i of an unbounded window sums i + 1 values over i + 2
    out = orc.windowed_attention(q, k, v, 1.0, sink=torch.zeros(1, dtype=F))
    assert torch.allclose(out[:, 0, 0], torch.tensor([sum(range(i + 1)) / (i + 2) for i in range(T)], dtype=F))
    # penalty r1 ln(1 + r2 d) with r1 = 1: weight of a key at distance d is 1 / (1 + r2 d)
    out = orc.windowed_attention(q, k, v, 1.0, r1=torch.ones(1, dtype=F), r2=torch.full((1,), 2.0, dtype=F))
    w = torch.tensor([1 / (1 + 2.0 * (3 - j)) for j in range(4)], dtype=F)
    assert math.isclose(float(out[3, 0, 0]), float((w * torch.arange(4, dtype=F)).sum() / w.sum()))


def test_oracle_mixed_heads_rotation_and_gru():
    T, D = 5, 4
    g = torch.Generator().manual_seed(0)
    q, k, v = (torch.randn(T, 2, D, generator=g, dtype=F) for _ in range(3))
    plain = orc.windowed_attention(q, k, v, 0.7)
    assert torch.allclose(orc.windowed_attention(q, k, v, 0.7, talk=torch.eye(2, dtype=F)), plain)
    swap = orc.windowed_attention(q, k, v, 0.7, talk=torch.tensor([[0.0, 1.0], [1.0, 0.0]], dtype=F))
    # swapped scores: head 0 weighs ITS values with head 1's scores
    assert torch.allclose(swap[:, 0], orc.windowed_attention(q[:, [1, 1]], k[:, [1, 0]], v[:, [0, 0]], 0.7)[:, 0])
    # rotation: a quarter turn of the first pair at position 1 when the pair's step is pi / 2; later coordinates pass
    x = torch.tensor([[1.0, 0.0, 5.0, 6.0]], dtype=F)
    y = orc.rotate_pairs(x, 1, 2, 1.0)     # base 1: every step is 1 radian
    assert torch.allclose(y, torch.tensor([[math.cos(1.0), math.sin(1.0), 5.0, 6.0]], dtype=F))
    dots = [float(orc.rotate_pairs(x, p, 4, 50.0)[0] @ orc.rotate_pairs(x, p + 3, 4, 50.0)[0]) for p in (0, 7, 100)]
    assert max(dots) - min(dots) < 1e-9        # the product of rotated vectors depends on the distance only
    # recurrent unit: z = 1/2 everywhere and a constant candidate c: S_t = c (1 - 2^-(t+1))
    zl, u = torch.zeros(4, 3, dtype=F), torch.full((4, 3), 1.5, dtype=F)
    assert torch.allclose(orc.min_gru_states(zl, u)[:, 0], torch.tensor([2.0 * (1 - 0.5 ** (t + 1)) for t in range(4)], dtype=F))
    assert torch.allclose(orc.gru_candidate(torch.tensor([-1.0, 0.0, 2.0], dtype=F)), torch.tensor([1 / (1 + math.e), 0.5, 2.5], dtype=F))

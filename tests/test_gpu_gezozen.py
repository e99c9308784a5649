"""Gezozen on the GPU against the float64 oracle (tests/gezozen_oracle.py): every mechanism alone (sigmoid top-k routing, head-wise
query/key preparation with norms, rotation in halves and stretched frequencies, the matrix-memory recurrence in its three uses fed
in portions through dirty state slots, a far key that only an undecayed memory keeps, the decay and read-out kernels), then the
executor through the engine's step function under different cuttings of the same tokens (whole prompts, token-by-token decoding,
portions down to two tokens, unequal batches, recycled cache blocks and state slots), window and page edges with inputs that make
a single key stand out, other sizes, random models, and greedy generation through the scheduler.  Small random models built here;
float32 mode is held to 2e-4 of the logits' spread, bfloat16 mode to 4e-2."""
import ctypes as C
import dataclasses
import json
import math
import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest

pytestmark = pytest.mark.gpu
ROOT = Path(__file__).resolve().parent.parent
TOL = {"float32": 2e-4, "bfloat16": 4e-2}


@pytest.fixture(scope="module")
def gpu():
    import torch
    import vllm_rust_amd as vmx
    assert torch.cuda.is_available()
    vmx.init(0)
    return vmx, torch


def rot(dims, base=500.0, **scaling):
    from vllm_rust_amd.gezozen import RotationSpec
    return RotationSpec(dims, base, dict(scaling) if scaling else None)


MOE = dict(mlp="moe", experts=5, top=2, expert_ff=20, shared_ff=28)


def delta_layer(**kw):
    from vllm_rust_amd.gezozen import GezozenLayerSpec
    d = dict(mixer="delta", heads=4, kv_heads=2, dim=10, vdim=14, conv=3, **MOE)
    d.update(kw)
    return GezozenLayerSpec(**d)


def gla_layer(**kw):
    from vllm_rust_amd.gezozen import GezozenLayerSpec
    d = dict(mixer="parallel", heads=6, kv_heads=2, dim=12, vdim=10, scale=0.4, softcap=7.0, rot=rot(8), r_heads=3, r_dim=10, r_vdim=6, tau=4.0,
             decay_rank=5, left_scale=0.7, right_scale=1.2, **MOE)
    d.update(kw)
    return GezozenLayerSpec(**d)


def ret_layer(**kw):
    from vllm_rust_amd.gezozen import GezozenLayerSpec
    d = dict(mixer="parallel_2", heads=4, kv_heads=2, dim=10, vdim=14, window=7, scale=0.35, rot=rot(6, 300.0, factor=4.0, original=16.0, fast=4.0, slow=1.0),
             r_heads=3, r_dim=8, r_vdim=12, decay=(0.8, 0.95, 0.995), r_rot=rot(8, 1000.0), left_scale=1.1, right_scale=0.6, **MOE)
    d.update(kw)
    return GezozenLayerSpec(**d)


def small_spec(layers=None, **kw):
    from vllm_rust_amd.gezozen import GezozenSpec
    layers = layers or [delta_layer(), gla_layer(mlp=None), ret_layer(top=1, shared_ff=0), delta_layer(heads=3, kv_heads=3, dim=7, vdim=5, conv=4, mlp=None),
                        gla_layer(heads=2, kv_heads=2, softcap=0.0, rot=rot(12), top=5)]
    d = dict(vocab=67, width=40, layers=layers, norm_eps=1e-5, norm_groups=2, postln_alpha=2.5)
    d.update(kw)
    return GezozenSpec(**d)


def sure_routing(spec):
    """The same model with every expert chosen (top = experts): long bfloat16 runs, where some router decision among hundreds is
    always a close call, then test everything but the choice."""
    return dataclasses.replace(spec, layers=[dataclasses.replace(l, top=l.experts) if l.mlp else l for l in spec.layers])


def build(spec, dtype="float32", seed=0, tweak=None, block_size=4, num_blocks=96, max_tokens=320, max_seqs=6):
    from vllm_rust_amd.engine import Engine
    from vllm_rust_amd.gezozen import GezozenForCausalLM, synthetic_weights
    ck = synthetic_weights(spec, seed)
    if tweak:
        tweak(ck)
    model = GezozenForCausalLM(spec, dtype=dtype, block_size=block_size, num_blocks=num_blocks, max_tokens=max_tokens, max_seqs=max_seqs)
    model.load_state(ck)
    return model, Engine(model), {k: v.double() for k, v in ck.items()}


def rel_err(got, want):
    """Difference of two logits arrays, row means removed, relative to the spread of the expected rows (worst row)."""
    g, w = np.asarray(got, np.float64), np.asarray(want, np.float64)
    d = g - w
    d = d - d.mean(-1, keepdims=True)
    return float((np.sqrt((d ** 2).mean(-1)) / (w.std(-1) + 1e-12)).max())


def routed(spec, dtype):
    """The model as it is in float32; in bfloat16 with every expert chosen (the choice itself is tested in float32, on single
    layers in bfloat16, and by the router's own test)."""
    return sure_routing(spec) if dtype == "bfloat16" else spec


def tokens_for(spec, n, seed, weights=None, dtype="bfloat16"):
    """n random token ids.  With the model's weights: the first draw on which no router decision of the oracle is a close call
    (relative gap above 2 % for bfloat16 runs, 0.01 % for float32 ones), since a decision that rounding can flip says nothing
    about the kernels."""
    margin = 0.02 if dtype == "bfloat16" else 1e-4
    from tests import gezozen_oracle as orc
    for attempt in range(200):
        toks = np.random.default_rng(seed + 1000 * attempt).integers(0, spec.vocab, n).tolist()
        if weights is None:
            return toks
        margins = []
        orc.forward(spec.to_config(), weights, toks, margins)
        if not margins or min(margins) > margin:
            return toks
    raise AssertionError("no token draw with safe router margins")


def oracle(spec, weights, toks):
    from tests import gezozen_oracle as orc
    lg, tr = orc.forward(spec.to_config(), weights, toks)
    return lg.numpy(), tr.numpy()


def feed(engine, seq_id, toks, cuts, finish=True):
    """Feed toks to one sequence in pieces of the given sizes (the last size repeats); logits of every position."""
    out, at, i = [], 0, 0
    while at < len(toks):
        n = min(cuts[min(i, len(cuts) - 1)], len(toks) - at)
        lg, _, _ = engine.step([(seq_id, toks[at:at + n], list(range(n)))])
        out.append(lg.cpu().numpy())
        at += n
        i += 1
    if finish:
        engine.finish(seq_id)
    return np.concatenate(out)


# ----------------------------------------------------------------------------- mechanisms alone

@pytest.mark.parametrize("E,top", [(4, 1), (16, 1), (5, 5), (70, 3), (256, 8), (1, 1)])
def test_sigmoid_router(gpu, E, top):
    _, torch = gpu
    from tests import gezozen_oracle as orc
    from vllm_rust_amd._lib import check, lib
    g = torch.Generator().manual_seed(E)
    h, w = torch.randn((23, 16), generator=g).double(), {"router": (3 * torch.randn((E, 16), generator=g)).double()}
    z = (h @ w["router"].T).float()
    z[5] = 0.25                                                   # every expert ties: the smallest indices win
    ids, s = orc.route(h, w, "", top)
    zc = z.cuda()
    wo, io = torch.empty(23, top, device="cuda"), torch.empty(23, top, dtype=torch.int32, device="cuda")
    check(lib.vmx_topk_sigmoid(zc.data_ptr(), wo.data_ptr(), io.data_ptr(), 23, E, top, 0, None))
    torch.cuda.synchronize()
    keep = [t for t in range(23) if t != 5]
    assert io.cpu()[keep].tolist() == ids[keep].tolist()
    assert float((wo.cpu()[keep].double() - s[keep]).abs().max()) < 1e-6   # scores as they are: not renormalised
    assert io.cpu()[5].tolist() == list(range(top)) and float((wo.cpu()[5] - 1 / (1 + math.exp(-0.25))).abs().max()) < 1e-6


@pytest.mark.parametrize("H,G,hd,rd,stretch,norms", [(4, 2, 12, 8, False, True), (3, 1, 10, 10, True, True), (8, 2, 64, 32, True, True), (2, 2, 7, 0, False, True),
                                                    (6, 3, 96, 48, False, False), (1, 1, 130, 64, True, True), (5, 5, 6, 2, False, False)])
@pytest.mark.parametrize("dtype", [0, 1])
@pytest.mark.parametrize("cached", [True, False])
def test_qk_prepare_head_by_head(gpu, H, G, hd, rd, stretch, norms, dtype, cached):
    _, torch = gpu
    from tests import gezozen_oracle as orc
    from vllm_rust_amd._lib import QkPrepareOpts, Rotation, check, lib
    T, vw, eps = 9, 20, 1e-5
    qw, kw_ = H * hd, G * hd
    g = torch.Generator().manual_seed(qw)
    q, k, v = (torch.randn(T, n, generator=g, dtype=torch.float64) for n in (qw, kw_, vw))
    qn, kn = ((1 + 0.2 * torch.randn(hd, generator=g, dtype=torch.float64)).to(torch.bfloat16) for _ in range(2))
    pos = torch.tensor([0, 1, 2, 3, 50, 51, 1000, 1001, 5000], dtype=torch.int32)
    slots = torch.tensor([5, 4, -1, 0, 1, 2, 11, 10, 7], dtype=torch.int32)
    rotd = dict(dims=rd, base=777.0, **({"scaling": dict(factor=4.0, original=64.0, fast=8.0, slow=1.0)} if stretch else {})) if rd else None
    fused = torch.cat([q, k, v], 1).float().cuda()
    ld = qw + kw_ + vw
    qo = torch.empty(T, qw, dtype=torch.float32, device="cuda")
    cdt = torch.float32 if dtype == 0 else torch.bfloat16
    kc, vc = torch.zeros(12, kw_, dtype=cdt, device="cuda"), torch.zeros(12, vw, dtype=cdt, device="cuda")
    ko = torch.zeros(T, kw_ + 3, dtype=torch.float32, device="cuda")
    steps, mul = None, 1.0
    if rd:
        sc = rotd.get("scaling") or {}
        r = Rotation(rd, 777.0, sc.get("factor", 0.0), sc.get("original", 0.0), sc.get("fast", 0.0), sc.get("slow", 0.0))
        buf, m = (C.c_float * (rd // 2))(), C.c_float()
        check(lib.vmx_rotation_steps(C.byref(r), buf, C.byref(m)))
        steps, mul = torch.tensor(list(buf), dtype=torch.float32, device="cuda"), m.value
    qnd, knd, posd, slotsd = qn.cuda(), kn.cuda(), pos.cuda(), slots.cuda()
    qm, km = 0.5, 1.0 / math.sqrt(hd)
    opts = QkPrepareOpts(1, 1, mul, qm, km, None if cached else ko.data_ptr(), kw_ + 3)
    check(lib.vmx_qk_prepare_ex(qo.data_ptr(), fused.data_ptr(), ld, qw, fused.data_ptr() + 4 * qw, ld, kw_, fused.data_ptr() + 4 * (qw + kw_) if cached else None,
                                ld, vw, qnd.data_ptr() if norms else None, knd.data_ptr() if norms else None, eps,
                                None if steps is None else steps.data_ptr(), rd, hd, posd.data_ptr(), slotsd.data_ptr() if cached else None,
                                kc.data_ptr() if cached else None, vc.data_ptr() if cached else None, dtype, T, C.byref(opts), None))
    torch.cuda.synchronize()
    qf, kf = q.float().double().reshape(T, H, hd), k.float().double().reshape(T, G, hd)
    if norms:
        qf, kf = orc.rms_unit(qf, eps) * qn.double(), orc.rms_unit(kf, eps) * kn.double()
    qf = torch.stack([orc.rotate_halves(qf[t], int(pos[t]), rotd) for t in range(T)]).reshape(T, qw) * qm
    kf = torch.stack([orc.rotate_halves(kf[t], int(pos[t]), rotd) for t in range(T)]).reshape(T, kw_) * km
    # angles are f32 products of a position and an f32 step: at position 5000 they carry an error of about 5000 * 2^-24
    tol = 1e-5 if not rd else 6e-3
    assert float((qo.cpu().double() - qf).abs().max()) < tol * 4
    if not cached:
        assert float((ko.cpu().double()[:, :kw_] - kf).abs().max()) < tol * 4 and float(ko[:, kw_:].abs().max()) == 0
        assert float(kc.abs().max()) == 0 and float(vc.abs().max()) == 0
        return
    for t in range(T):
        s = int(slots[t])
        if s >= 0:
            assert float((kc[s].cpu().double() - kf[t]).abs().max()) < (tol * 4 if dtype == 0 else 0.04)
            assert float((vc[s].cpu().double() - v[t].float().double()).abs().max()) < (1e-6 if dtype == 0 else 0.04)
    assert float(kc[3].abs().max()) == 0 and float(kc[6].abs().max()) == 0   # untouched rows (slot -1 wrote nothing)


def _run_recurrence(torch, mode, q, k, v, g, beta, portions, slot_of, qk_heads, q_mul=1.0):
    """vmx_matrix_memory_recurrence over several sequences fed in unequal portions through slots that start full of NaN.
    q, k: lists of [n, qk_heads, D]; v: [n, H, V]; g: per mode [n, H, D] (channel), [n, H] (head) or [H] (constant)."""
    from vllm_rust_amd._lib import check, lib
    H, V, D = v[0].shape[1], v[0].shape[2], q[0].shape[2]
    nslots = max(slot_of) + 2
    state = torch.full((lib.vmx_gated_delta_rule_state_bytes(nslots, H, D, V) // 4,), float("nan"), dtype=torch.float32, device="cuda")
    lens = [x.shape[0] for x in q]
    got, fed = [[] for _ in lens], [0] * len(lens)
    i32 = lambda a: torch.tensor(a, dtype=torch.int32, device="cuda")
    gconst = g.float().cuda() if mode == "const" else None
    for step in range(max(len(p) for p in portions)):
        parts, starts, slots, posn, owners = [], [0], [], [], []
        for s, n in enumerate(lens):
            if step < len(portions[s]) and fed[s] < n:
                c = min(portions[s][step], n - fed[s])
                a, b = fed[s], fed[s] + c
                cols = [q[s][a:b].reshape(c, -1), k[s][a:b].reshape(c, -1), v[s][a:b].reshape(c, -1)]
                if mode != "const":
                    cols.append(g[s][a:b].reshape(c, -1))
                if beta is not None:
                    cols.append(beta[s][a:b].reshape(c, -1))
                parts.append(torch.cat(cols, 1))
                posn += list(range(a, b))
                starts.append(starts[-1] + c)
                slots.append(slot_of[s])
                owners.append((s, c))
                fed[s] = b
        x = torch.cat(parts).float().cuda()
        T, ld = x.shape
        o = torch.empty(T, H * V, dtype=torch.float32, device="cuda")
        P, S, L = i32(posn), i32(starts), i32(slots)
        oq, ok, ov = 0, qk_heads * D, 2 * qk_heads * D
        og = ov + H * V
        gw = 0 if mode == "const" else (H * D if mode == "channel" else H)
        ob = og + gw
        check(lib.vmx_matrix_memory_recurrence(o.data_ptr(), H * V, x.data_ptr() + 4 * oq, ld, q_mul, x.data_ptr() + 4 * ok, ld, x.data_ptr() + 4 * ov, ld,
                                               gconst.data_ptr() if mode == "const" else x.data_ptr() + 4 * og, 0 if mode == "const" else ld,
                                               0 if mode == "channel" else 1, None if beta is None else x.data_ptr() + 4 * ob, ld, state.data_ptr(),
                                               P.data_ptr(), S.data_ptr(), L.data_ptr(), len(slots), H, qk_heads, D, V, None))
        torch.cuda.synchronize()
        at = 0
        for s, c in owners:
            got[s].append(o[at:at + c].cpu())
            at += c
    assert fed == lens
    return [torch.cat(x).double().reshape(n, H, V) for x, n in zip(got, lens)]


@pytest.mark.parametrize("mode", ["channel", "const", "head_delta"])
@pytest.mark.parametrize("H,G,D,V", [(2, 1, 32, 32), (3, 3, 5, 7), (4, 2, 64, 40), (6, 6, 130, 16), (1, 1, 16, 1)])
def test_matrix_memory_in_portions_through_dirty_slots(gpu, mode, H, G, D, V):
    """The three uses of the recurrence kernel (a decay per key channel with the plain write; a constant per head with the plain
    write; a decay per head and token with the delta rule over grouped query/key heads): three sequences of unequal length in
    portions of 1 .. 90 rows, against the oracle's recurrence over the whole sequences."""
    _, torch = gpu
    from tests import gezozen_oracle as orc
    if mode != "head_delta":
        G = H
    gen = torch.Generator().manual_seed(H * D + V)
    lens = [131, 1, 47]
    rn = lambda *s: torch.randn(*s, generator=gen, dtype=torch.float64).float().double()
    q, k, v = [rn(n, G, D) for n in lens], [rn(n, G, D) * D ** -0.5 for n in lens], [rn(n, H, V) for n in lens]
    beta = None
    if mode == "channel":
        g = [torch.sigmoid(rn(n, H, D) + 2) for n in lens]
    elif mode == "const":
        g = torch.tensor([0.7, 0.9, 0.97, 0.99, 0.995, 1.0][:H], dtype=torch.float64).float().double()
    else:
        k = [x / x.norm(dim=-1, keepdim=True) for x in k]
        g, beta = [torch.sigmoid(rn(n, H) + 2) for n in lens], [torch.sigmoid(rn(n, H)) for n in lens]
    k = [x.float().double() for x in k]
    g = [x.float().double() for x in g] if mode != "const" else g
    beta = None if beta is None else [x.float().double() for x in beta]
    got = _run_recurrence(torch, mode, q, k, v, g, beta, [[90, 1, 1, 37, 2], [1], [2, 3, 40, 1, 1]], [3, 0, 4], G, q_mul=0.75)
    for s, n in enumerate(lens):
        if mode == "head_delta":
            rep = H // G
            want = orc.delta_rule_memory(q[s].repeat_interleave(rep, 1) * 0.75, k[s].repeat_interleave(rep, 1), v[s], g[s], beta[s])
        else:
            dec = g[s] if mode == "channel" else g.reshape(1, H, 1).expand(n, H, D)
            want = orc.decayed_outer_memory(q[s] * 0.75, k[s], v[s], dec)
        assert float((got[s] - want).abs().max()) < 3e-5 * max(1.0, float(want.abs().max())), (mode, s)


def test_matrix_memory_keeps_a_far_key(gpu):
    """Decay 1 on one head, 0.9 on the other: a key written at position 5 and asked for 290 tokens later (in a later portion)
    comes back whole from the first and is gone from the second; every other key is orthogonal to the question."""
    _, torch = gpu
    n, D, V = 300, 16, 8
    gen = torch.Generator().manual_seed(0)
    k = torch.zeros(n, 2, D, dtype=torch.float64)
    k[:, :, 1:] = torch.randn(n, 2, D - 1, generator=gen, dtype=torch.float64).float().double()
    k[5, :, 0] = 1.0
    v = torch.randn(n, 2, V, generator=gen, dtype=torch.float64).float().double()
    q = torch.zeros(n, 2, D, dtype=torch.float64)
    q[:, :, 0] = 1.0
    got = _run_recurrence(torch, "const", [q], [k], [v], torch.tensor([1.0, 0.9], dtype=torch.float64), None, [[4, 100, 1, 150, 45]], [1], 2)[0]
    assert float(got[:5].abs().max()) == 0
    for t in (5, 6, 104, 105, 295, 299):
        assert float((got[t, 0] - v[5, 0]).abs().max()) < 1e-5
        assert float((got[t, 1] - v[5, 1] * 0.9 ** (t - 5)).abs().max()) < 1e-5


def test_decay_and_read_out_kernels(gpu):
    _, torch = gpu
    from tests import gezozen_oracle as orc
    from vllm_rust_amd._lib import check, lib
    gen = torch.Generator().manual_seed(4)
    z = (torch.randn(7, 50, generator=gen) * 6).cuda()
    want = torch.sigmoid(z.cpu().double()[:, :44]) ** (1 / 12.0)
    check(lib.vmx_sigmoid_root_decay(z.data_ptr(), 50, 7, 44, 12.0, None))
    torch.cuda.synchronize()
    assert float((z.cpu().double()[:, :44] - want).abs().max()) < 1e-6
    for H, V, gain in ((3, 10, True), (2, 70, False), (5, 1, True), (1, 200, True)):
        o = torch.randn(6, H * V, generator=gen).cuda() * 3
        gate = torch.randn(6, H * V + 4, generator=gen).cuda()
        w = (1 + 0.2 * torch.randn(V, generator=gen)).to(torch.bfloat16).cuda()
        y = torch.empty(6, H * V, dtype=torch.float32, device="cuda")
        check(lib.vmx_head_rms_gate_ex(y.data_ptr(), 0, o.data_ptr(), H * V, w.data_ptr() if gain else None, gate.data_ptr(), H * V + 4, 1, 1e-5, 6, H, V, None))
        torch.cuda.synchronize()
        ref = orc.rms_unit(o.cpu().double().reshape(6, H, V), 1e-5) * (w.cpu().double() if gain else 1.0)
        ref = ref.reshape(6, H * V) * orc.silu(gate.cpu().double()[:, :H * V])
        assert float((y.cpu().double() - ref).abs().max()) < 1e-5


# ----------------------------------------------------------------------------- the executor through the engine

@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_layers_and_logits_against_the_oracle(gpu, dtype):
    spec = routed(small_spec(), dtype)
    model, eng, w = build(spec, dtype)
    toks = tokens_for(spec, 41, 1, w, dtype)
    lg, _, tr = eng.step([("a", toks, list(range(len(toks))))], layer_trace=True)
    want, wtr = oracle(spec, w, toks)
    assert tr.shape[0] == len(spec.layers) == 5
    for r in range(tr.shape[0]):
        assert rel_err(tr[r].cpu().numpy(), wtr[r]) < TOL[dtype], f"layer {r}"
    assert rel_err(lg.cpu().numpy(), want) < TOL[dtype]


@pytest.mark.parametrize("kind", ["delta", "parallel", "parallel_2"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_every_layer_kind_alone(gpu, dtype, kind):
    """One layer of each kind with and without its feed-forward, one norm group and several: the stream after the layer."""
    make = {"delta": delta_layer, "parallel": gla_layer, "parallel_2": ret_layer}[kind]
    for groups, layer in ((1, make()), (5, make(mlp=None)), (4, make(top=1, shared_ff=0, experts=3))):
        spec = small_spec(layers=[layer], norm_groups=groups)
        model, eng, w = build(spec, dtype)
        toks = tokens_for(spec, 26, 2, w, dtype)
        lg, _, tr = eng.step([("a", toks, list(range(26)))], layer_trace=True)
        want, wtr = oracle(spec, w, toks)
        assert rel_err(tr[0].cpu().numpy(), wtr[0]) < TOL[dtype], (kind, groups)
        assert rel_err(lg.cpu().numpy(), want) < TOL[dtype], (kind, groups)
        model.close()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_prompt_decode_and_portions_agree(gpu, dtype):
    spec = routed(small_spec(), dtype)
    model, eng, w = build(spec, dtype)
    toks = tokens_for(spec, 53, 2, w, dtype)
    want, _ = oracle(spec, w, toks)
    for cuts in ([53], [1], [2], [3], [7, 16], [16, 1], [20, 2, 1]):
        got = feed(eng, "s", toks, cuts)
        assert rel_err(got, want) < TOL[dtype], f"cuts {cuts}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_unequal_batches_and_recycled_blocks_and_slots(gpu, dtype):
    """Three requests of unequal length in one batch, then decoded together while the short ones finish early; five generations of
    requests through 3 state slots and few blocks, freed blocks and slots handed out again in another order."""
    spec = routed(small_spec(), dtype)
    model, eng, w = build(spec, dtype, num_blocks=40, max_seqs=3)
    for gen in range(5):
        lens = [(29, 6), (3, 2), (14, 9)]
        reqs = {f"g{gen}r{i}": tokens_for(spec, n + d, 100 * gen + i, w, dtype) for i, (n, d) in enumerate(lens)}
        want = {k: oracle(spec, w, t)[0] for k, t in reqs.items()}
        got = {k: [] for k in reqs}
        lg, _, _ = eng.step([(k, reqs[k][:n], list(range(n))) for k, (n, _) in zip(reqs, lens)])
        at = 0
        for k, (n, _) in zip(reqs, lens):
            got[k].append(lg[at:at + n].cpu().numpy())
            at += n
        fed = {k: n for k, (n, _) in zip(reqs, lens)}
        while True:
            live = [k for k in reqs if fed[k] < len(reqs[k])]
            if not live:
                break
            lg, _, _ = eng.step([(k, [reqs[k][fed[k]]], [0]) for k in live])
            for j, k in enumerate(live):
                got[k].append(lg[j:j + 1].cpu().numpy())
                fed[k] += 1
                if fed[k] == len(reqs[k]):
                    eng.finish(k)     # leaves the batch early; its blocks and slot go back
        for k in reqs:
            assert rel_err(np.concatenate(got[k]), want[k]) < TOL[dtype], k
    assert len(eng.blocks.free) == 40 and len(eng.states.free) == 3


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("window,bs", [(1, 1), (2, 4), (3, 3), (4, 4), (5, 16), (8, 8), (16, 16), (17, 16)])
def test_small_windows_on_page_sizes(gpu, dtype, window, bs):
    """Windows of a few keys (each visible key carries weight): a key one step too far or too near moves the logits."""
    spec = routed(small_spec(layers=[ret_layer(window=window), delta_layer(mlp=None), ret_layer(window=window + 1, mlp=None)]), dtype)
    model, eng, w = build(spec, dtype, block_size=bs, num_blocks=max(24, 400 // bs))
    toks = tokens_for(spec, 45, window, w, dtype)
    want, _ = oracle(spec, w, toks)
    assert rel_err(feed(eng, "a", toks, [45]), want) < TOL[dtype]
    assert rel_err(feed(eng, "b", toks, [20, 1]), want) < TOL[dtype]
    assert rel_err(feed(eng, "c", toks, [5, 2]), want) < TOL[dtype]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("sizes", ["any", "eights"])
def test_sharp_attention_over_300_tokens_and_long_decoding(gpu, dtype, sizes):
    """Queries scaled up so that single keys decide rows, a window of 70 keys over page borders and causal attention over all 300
    tokens, slow decays in the memories, 220 tokens as a prompt and 80 decoded one by one; every expert chosen (no close calls)."""
    def sharpen(ck):
        for k in ck:
            if k.endswith("left.q.norm"):
                ck[k] = (ck[k].float() * 3).to(ck[k].dtype)
            if k.endswith("A_log"):
                ck[k] = (ck[k].float() - 3).to(ck[k].dtype)       # decays close to 1: old writes stay in the delta rule's memory
    slow = (0.999, 0.99, 1.0)
    if sizes == "any":
        layers = [ret_layer(window=70, decay=slow), gla_layer(tau=64.0), delta_layer(mlp=None)]
    else:    # multiples of 8: the matrix-core forms in bfloat16, windows over several key tiles
        layers = [ret_layer(window=70, dim=16, vdim=24, rot=rot(8), decay=slow, r_dim=16, r_vdim=16, r_rot=rot(16, 1e4)),
                  gla_layer(dim=32, vdim=8, rot=rot(32, 1e4), tau=64.0, r_dim=32, r_vdim=32), delta_layer(mlp=None, dim=32, vdim=32)]
    spec = sure_routing(small_spec(layers=layers))
    model, eng, w = build(spec, dtype, tweak=sharpen, block_size=16, num_blocks=64, max_tokens=512)
    toks = tokens_for(spec, 300, 9)
    want, _ = oracle(spec, w, toks)
    assert rel_err(feed(eng, "a", toks, [220, 1]), want) < TOL[dtype]
    assert rel_err(feed(eng, "b", toks, [300]), want) < TOL[dtype]


def _attention_op(torch, q, k, v, scale, cap, window, block_size, dtype, runs, seed=1, pos0=0):
    """vmx_window_attention for ONE sequence whose blocks are scattered over a larger cache; the last T - pos0 positions are the
    queries (pos0 > 0: earlier rows are already cached).  runs: hand the operator seq_starts (matrix-core forms where sizes and
    cache allow); runs == "split": also a workspace, so that a run's keys are dealt to several workgroups and merged."""
    from vllm_rust_amd._lib import check, lib
    T, H, D = q.shape
    G, V = k.shape[1], v.shape[2]
    nb = (T + block_size - 1) // block_size
    perm = np.random.default_rng(seed).permutation(nb + 7)[:nb].astype(np.int32)
    cdt = torch.float32 if dtype == 0 else torch.bfloat16
    kc = torch.full(((nb + 7) * block_size, G * D), float("nan"), dtype=torch.float32)
    vc = torch.full(((nb + 7) * block_size, G * V), float("nan"), dtype=torch.float32)
    pos = np.arange(T)
    rows = perm[pos // block_size] * block_size + pos % block_size
    kc[rows], vc[rows] = k.reshape(T, G * D).float(), v.reshape(T, G * V).float()
    kc, vc = kc.to(cdt).cuda(), vc.to(cdt).cuda()
    n = T - pos0
    out = torch.empty((n, H * V), dtype=torch.float32, device="cuda")
    qd = q[pos0:].reshape(n, H * D).float().contiguous().cuda()
    bt, sid = torch.from_numpy(perm[None]).cuda(), torch.zeros(n, dtype=torch.int32, device="cuda")
    pid = torch.arange(pos0, T, dtype=torch.int32, device="cuda")
    st = torch.tensor([0, n], dtype=torch.int32, device="cuda")
    ws = torch.empty(lib.vmx_window_attention_workspace_bytes(n, H, V) // 4, dtype=torch.float32, device="cuda")
    check(lib.vmx_window_attention(out.data_ptr(), 0, qd.data_ptr(), H * D, kc.data_ptr(), vc.data_ptr(), dtype, bt.data_ptr(), nb, sid.data_ptr(),
                                   pid.data_ptr(), None, None, 0, scale, cap, window, 0, n, H, G, D, V, block_size, st.data_ptr() if runs else None,
                                   1 if runs else 0, ws.data_ptr() if runs == "split" else None, ws.numel() * 4, None))
    torch.cuda.synchronize()
    return out.cpu().double().reshape(n, H, V)


FORMS = [(0, False), (1, False), (1, True), (1, "split")]   # (cache dtype, runs): f32 vector, bf16 vector, matrix cores, + key shares


@pytest.mark.parametrize("form", FORMS)
@pytest.mark.parametrize("window,bs,cap", [(40, 16, 0.0), (64, 16, 30.0), (65, 8, 30.0), (17, 5, 0.0), (96, 16, 20.0)])
def test_attention_needle_at_the_window_edge_and_far_back(gpu, form, window, bs, cap):
    """One key carries a score far above the rest.  Queries at distance window - 1 (the last that see it) and window (the first
    that do not), in a prompt and as single decoded rows, on several page sizes, with and without the soft cap (which flattens the
    needle's score to the cap, still far above the others); without a window the needle stays visible from 292 keys away."""
    _, torch = gpu
    from tests import gezozen_oracle as orc
    dtype, runs = form
    H, G, D = 4, 2, 16
    T = 330
    g = torch.Generator().manual_seed(3)
    q, k, v = (torch.randn(s, generator=g, dtype=torch.float64) for s in ((T, H, D), (T, G, D), (T, G, D)))
    q, k = q * 0.2, k * 0.2
    needle = 37
    d = torch.randn(G, D, generator=g, dtype=torch.float64).sign()
    k[needle] = d                                     # score 16 against a query along d; every other score is of order 1
    for i in (needle + window - 1, needle + window, T - 1):
        q[i] = d.repeat_interleave(H // G, dim=0)
    bfr = lambda t: t.to(torch.bfloat16).double()
    q, k, v = bfr(q), bfr(k), bfr(v)
    tol = 2e-5 if dtype == 0 else 8e-3
    vn = v[needle].repeat_interleave(H // G, dim=0)
    for win in (window, 0):
        want = orc.softmax_attention(q, k, v, 1.0, cap, win)
        got = _attention_op(torch, q, k, v, 1.0, cap, win, bs, dtype, runs)
        assert float((got - want).abs().max()) < tol * max(1.0, float(want.abs().max()))
        assert float((want[needle + window - 1] - vn).abs().max()) < 0.2            # the needle decides the row just inside
        if win:
            assert float((want[needle + window] - vn).abs().max()) > 0.2            # and is gone just outside
        else:
            assert float((want[T - 1] - vn).abs().max()) < 0.2                      # no window: still there at the end
        for i in (needle + window - 1, needle + window, T - 1):   # the same rows decoded alone over the cached keys
            one = _attention_op(torch, q[:i + 1], k[:i + 1], v[:i + 1], 1.0, cap, win, bs, dtype, runs, pos0=i)
            assert float((one[0] - want[i]).abs().max()) < tol * max(1.0, float(want.abs().max()))


OTHER_SIZES = {
    "one layer of each": dict(layers=[delta_layer(), gla_layer(), ret_layer()]),
    "reverse order": dict(layers=[ret_layer(), gla_layer(), delta_layer()]),
    "alpha 1, one group": dict(postln_alpha=1.0, norm_groups=1),
    "many groups": dict(norm_groups=8),
    "one head": dict(layers=[delta_layer(heads=1, kv_heads=1), gla_layer(heads=1, kv_heads=1, r_heads=1), ret_layer(heads=1, kv_heads=1, r_heads=1, decay=(0.9,))]),
    "equal head counts": dict(layers=[delta_layer(heads=4, kv_heads=4), gla_layer(heads=4, kv_heads=4), ret_layer(heads=2, kv_heads=2)]),
    "many heads per key head": dict(layers=[delta_layer(heads=8, kv_heads=1, dim=8, vdim=8), gla_layer(heads=10, kv_heads=2, dim=8, rot=rot(8)),
                                            ret_layer(heads=12, kv_heads=2, dim=8, vdim=8, rot=rot(8))]),
    "sizes of 8s": dict(layers=[delta_layer(heads=4, kv_heads=2, dim=32, vdim=64), gla_layer(heads=8, kv_heads=2, dim=32, vdim=64, rot=rot(16), r_dim=32, r_vdim=64),
                                ret_layer(heads=8, kv_heads=4, dim=64, vdim=32, window=40, rot=rot(32, 1e4, factor=4.0, original=32.0, fast=8.0, slow=1.0),
                                          r_dim=64, r_vdim=32, r_rot=rot(64, 1e6))], width=64),
    "odd sizes": dict(layers=[delta_layer(heads=3, kv_heads=1, dim=7, vdim=5, conv=2), gla_layer(heads=3, kv_heads=3, dim=7, vdim=3, rot=rot(2), r_heads=2, r_dim=5, r_vdim=9, decay_rank=1),
                              ret_layer(heads=2, kv_heads=1, dim=6, vdim=5, rot=rot(2), r_heads=1, r_dim=6, r_vdim=1, r_rot=rot(2), decay=(0.5,))], width=34),
    "no rotation, no window, no cap": dict(layers=[ret_layer(rot=rot(0), r_rot=rot(0), window=0), gla_layer(rot=rot(0), softcap=0.0)]),
    "full rotation, unstretched": dict(layers=[ret_layer(rot=rot(10), r_rot=rot(8)), gla_layer(rot=rot(12))]),
    "window and cap change sides": dict(layers=[ret_layer(softcap=5.0, window=0), gla_layer(window=6, softcap=0.0)]),
    "wide values": dict(layers=[gla_layer(dim=16, vdim=136, rot=rot(16)), ret_layer(dim=8, vdim=200, rot=rot(4))]),
    "key size 130": dict(layers=[gla_layer(dim=130, vdim=8, rot=rot(64), r_dim=130), delta_layer(heads=2, kv_heads=1, dim=132)]),
    "one tap": dict(layers=[delta_layer(conv=1), delta_layer(conv=9)]),
    "one expert": dict(layers=[delta_layer(experts=1, top=1), gla_layer(experts=2, top=2, shared_ff=0)]),
    "many experts": dict(layers=[delta_layer(experts=40, top=4, expert_ff=8), ret_layer(experts=17, top=1, shared_ff=8)]),
    "unit scales": dict(layers=[gla_layer(left_scale=1.0, right_scale=1.0, tau=1.0), ret_layer(left_scale=1.0, right_scale=1.0, decay=(1.0, 1.0, 1.0))]),
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(OTHER_SIZES))
def test_other_sizes(gpu, dtype, name):
    spec = routed(small_spec(**OTHER_SIZES[name]), dtype)
    model, eng, w = build(spec, dtype)
    toks = tokens_for(spec, 37, 4, w, dtype)
    want, wtr = oracle(spec, w, toks)
    lg, _, tr = eng.step([("a", toks, list(range(37)))], layer_trace=True)
    assert tr.shape[0] == len(spec.layers)
    assert rel_err(tr[-1].cpu().numpy(), wtr[-1]) < TOL[dtype]
    assert rel_err(lg.cpu().numpy(), want) < TOL[dtype]
    eng.finish("a")
    assert rel_err(feed(eng, "b", toks, [30, 1]), want) < TOL[dtype]
    assert rel_err(feed(eng, "c", toks, [2]), want) < TOL[dtype]


def random_spec(rng):
    layers = []
    pick = lambda *a: a[int(rng.integers(0, len(a)))]
    for _ in range(int(rng.integers(1, 6))):
        G = int(rng.integers(1, 4))
        H = G * int(rng.integers(1, 5))
        mult8 = rng.random() < 0.5
        D = int(rng.integers(1, 6)) * 8 if mult8 else 2 * int(rng.integers(2, 30))
        V = int(rng.integers(1, 6)) * 8 if mult8 else int(rng.integers(3, 70))
        E = int(rng.integers(1, 9))
        ff = dict(mlp="moe", experts=E, top=int(rng.integers(1, E + 1)), expert_ff=int(rng.integers(4, 40)), shared_ff=int(pick(0, 8, 24))) if rng.random() < 0.75 \
            else dict(mlp=None)
        kind = pick("delta", "parallel", "parallel_2")
        if kind == "delta":
            layers.append(delta_layer(heads=H, kv_heads=G, dim=D, vdim=V, conv=int(rng.integers(1, 6)), **ff))
            continue

        def any_rot(d):
            dims = 2 * int(rng.integers(0, d // 2 + 1))
            if dims and rng.random() < 0.5:
                return rot(dims, float(pick(100.0, 1e4, 1e6)), factor=float(pick(2.0, 4.0, 16.0)), original=float(pick(16, 64, 2048)), fast=float(pick(4.0, 32.0)),
                           slow=float(pick(0.5, 1.0, 2.0)))
            return rot(dims, float(pick(100.0, 1e4, 1e6)))
        RH, RD, RV = int(rng.integers(1, 5)), 2 * int(rng.integers(1, 20)), int(rng.integers(4, 40))   # a norm over 1 .. 3 numbers turns rounding into sign flips
        common = dict(heads=H, kv_heads=G, dim=D, vdim=V, scale=float(rng.uniform(0.1, 0.6)), rot=any_rot(D), r_heads=RH, r_dim=RD, r_vdim=RV,
                      left_scale=float(rng.uniform(0.3, 1.2)), right_scale=float(rng.uniform(0.3, 1.2)), **ff)
        if kind == "parallel":
            layers.append(gla_layer(softcap=float(pick(4.0, 30.0)), tau=float(pick(1.0, 4.0, 16.0)), decay_rank=int(rng.integers(1, 9)), **common))
        else:
            layers.append(ret_layer(window=int(pick(1, 2, 5, 16, 33, 64)), decay=tuple(float(1 - 2.0 ** -rng.uniform(1, 9)) for _ in range(RH)), r_rot=any_rot(RD),
                                    **common))
    groups = int(pick(1, 2, 4))
    width = groups * (int(rng.integers(2, 8)) * 4 if rng.random() < 0.5 else int(rng.integers(5, 30)))
    return small_spec(layers=layers, width=width, vocab=int(rng.integers(20, 300)), norm_groups=groups, postln_alpha=float(pick(1.0, 2.0, 3.5)),
                      norm_eps=float(pick(1e-6, 1e-5)))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", range(12))
def test_random_models(gpu, dtype, seed):
    """Models drawn at random (layer order, head counts, sizes, windows, caps, rotations, decays, experts) on random page sizes: two
    unequal requests decoding together, a third fed in portions."""
    rng = np.random.default_rng(seed)
    spec = routed(random_spec(rng), dtype)
    bs = int(rng.choice([1, 3, 4, 8, 16]))
    model, eng, w = build(spec, dtype, seed=seed, block_size=bs, num_blocks=600 // bs + 8)
    ta, tb, tc = tokens_for(spec, 75, seed, w, dtype), tokens_for(spec, 33, seed + 50, w, dtype), tokens_for(spec, 60, seed + 99, w, dtype)
    wa, wb, wc = (oracle(spec, w, t)[0] for t in (ta, tb, tc))
    lg, _, _ = eng.step([("a", ta[:60], list(range(60))), ("b", tb[:20], list(range(20)))])
    ga, gb = [lg[:60].cpu().numpy()], [lg[60:].cpu().numpy()]
    for i in range(15):
        ent = [("a", [ta[60 + i]], [0])] + ([("b", [tb[20 + i]], [0])] if i < 13 else [])
        lg, _, _ = eng.step(ent)
        ga.append(lg[:1].cpu().numpy())
        if i < 13:
            gb.append(lg[1:2].cpu().numpy())
        if i == 12:
            eng.finish("b")
    assert rel_err(np.concatenate(ga), wa) < TOL[dtype]
    assert rel_err(np.concatenate(gb), wb) < TOL[dtype]
    assert rel_err(feed(eng, "c", tc, [int(rng.integers(2, 20)), int(rng.integers(1, 9))]), wc) < TOL[dtype]


def test_greedy_generation_through_the_scheduler(gpu):
    """Engine.generate (scheduler, block pressure, prompt portions, greedy ids from the executor) against the oracle's argmax
    continuation; sampled generation runs and stays in the vocabulary."""
    from vllm_rust_amd.engine import SamplingParams
    spec = small_spec()
    model, eng, w = build(spec, "float32", num_blocks=30, max_seqs=3)
    prompts = [tokens_for(spec, n, 70 + n) for n in (9, 23, 4, 15, 2)]
    outs = eng.generate(prompts, SamplingParams(max_new_tokens=8), prefill_chunk=6)
    for p, o in zip(prompts, outs):
        seq = list(p)
        for t in o:
            margins = []
            from tests import gezozen_oracle as orc
            lg = orc.forward(spec.to_config(), w, seq, margins)[0].numpy()
            if min(margins) < 1e-4:
                break                         # a router decision within rounding: the continuation may differ legitimately
            top2 = np.sort(lg[-1])[-2:]
            if top2[1] - top2[0] > 1e-3:      # a tie within rounding says nothing
                assert int(np.argmax(lg[-1])) == t
            seq.append(t)
    assert len(eng.blocks.free) == 30 and len(eng.states.free) == 3
    outs = eng.generate(prompts[:3], SamplingParams(temperature=0.9, top_k=20, top_p=0.9, max_new_tokens=5, seed=3))
    assert all(len(o) == 5 and all(0 <= t < spec.vocab for t in o) for o in outs)


def _write_checkpoint(tmp_path, spec, seed=0):
    from safetensors.torch import save_file
    from vllm_rust_amd.gezozen import synthetic_weights
    ck = synthetic_weights(spec, seed)
    d = tmp_path / "model"
    d.mkdir()
    (d / "config.json").write_text(json.dumps(spec.to_config()))
    import torch
    extra = {f"l{i}.norm2": torch.ones(spec.width, dtype=torch.bfloat16) for i, l in enumerate(spec.layers) if l.mlp is None}   # a file may carry them: skipped
    save_file({k: v.contiguous() for k, v in {**ck, **extra}.items()}, str(d / "model.safetensors"))
    return d, {k: v.double() for k, v in ck.items()}


def test_registry_and_command_line_tools(gpu, tmp_path):
    """A checkpoint directory written here: the registry picks the class from config.json and reads the decay projection's inner
    size off the checkpoint; bin/trace_run replays a trace (a prompt, a portion, decode steps of two requests, an early finisher)
    in both modes; bin/generate continues greedily."""
    from vllm_rust_amd.engine import Engine
    from vllm_rust_amd.models import architecture_of, load_model
    spec = sure_routing(small_spec())        # one checkpoint for both modes
    d, w = _write_checkpoint(tmp_path, spec)
    assert architecture_of(d) == "Gezozen"
    model = load_model(d, dtype="float32", max_tokens=128, max_seqs=4, block_size=8)
    assert model.spec.to_config() == spec.to_config() and [l.decay_rank for l in model.spec.layers] == [0, 5, 0, 0, 5]
    ta, tb = tokens_for(spec, 30, 1), tokens_for(spec, 12, 2)
    wa, wb = oracle(spec, w, ta)[0], oracle(spec, w, tb)[0]
    lg, _, _ = Engine(model).step([("x", ta, [29])])
    assert rel_err(lg.cpu().numpy(), wa[29:30]) < TOL["float32"]
    model.close()
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": ta[:20], "want": [0, 19]}, {"id": "b", "tokens": tb[:10], "want": [9]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": [ta[20]], "want": [0]}, {"id": "b", "tokens": [tb[10]], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": [ta[21]], "want": [0]}, {"id": "b", "tokens": [tb[11]], "want": [0]}], "end": ["b"]},
             {"step": 3, "entries": [{"id": "a", "tokens": ta[22:30], "want": [7]}], "end": ["a"]}]
    for dtype in ("float32", "bfloat16"):
        out = tmp_path / f"out_{dtype}"
        r = subprocess.run([sys.executable, str(ROOT / "bin" / "trace_run"), "--model", str(d), "--dtype", dtype, "--out", str(out), "--max-tokens", "64"],
                           input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=300)
        assert r.returncode == 0, r.stderr
        assert [l for l in r.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(4)]
        rd = lambda i: np.fromfile(out / f"{i}.f32", dtype="<f4").reshape(-1, spec.vocab)
        assert rel_err(rd(0), np.stack([wa[0], wa[19], wb[9]])) < TOL[dtype]
        assert rel_err(rd(1), wa[20:21]) < TOL[dtype]
        assert rel_err(rd(2), np.stack([wa[21], wb[11]])) < TOL[dtype]
        assert rel_err(rd(3), wa[29:30]) < TOL[dtype]
    r = subprocess.run([sys.executable, str(ROOT / "bin" / "generate"), "--model", str(d), "--dtype", "float32", "--prompt", ",".join(map(str, ta[:9])),
                        "--max-new-tokens", "4"], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr
    ids = [int(t) for t in r.stdout.strip().splitlines()[-1].split(",")]
    assert len(ids) == 4 and all(0 <= t < spec.vocab for t in ids)

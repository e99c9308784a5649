"""Vokepel on the GPU against the float64 oracle (tests/vokepel_oracle.py): every mechanism alone (query/key preparation with
whole-row norms and pair rotation, attention with sink / distance penalty / mixed heads / element-wise gate on scattered pages in
every kernel form, the gated recurrent unit with carried state), then the executor through the engine's step function under
different cuttings of the same tokens (whole prompts, token-by-token decoding, portions down to two tokens, unequal batches,
recycled cache blocks and state slots), window and page edges with inputs that make a single key stand out, other sizes, random
models, and greedy generation through the scheduler.  Small random models built here; float32 mode is held to 2e-4 of the logits'
spread, bfloat16 mode to 4e-2."""
import dataclasses
import json
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


def talk_layer(**kw):
    from vllm_rust_amd.vokepel import VokepelLayerSpec
    d = dict(mixer="attention", heads=6, kv_heads=2, dim=12, vdim=12, window=7, scale=0.4, softcap=9.0, mlp="dense", ff=56)
    d.update(kw)
    if "dim" in kw and "vdim" not in kw:
        d["vdim"] = d["dim"]
    return VokepelLayerSpec(**d)


def pair_layer(**kw):
    from vllm_rust_amd.vokepel import VokepelLayerSpec
    d = dict(mixer="parallel", heads=4, kv_heads=2, dim=10, vdim=14, window=5, scale=0.35, rot_dims=6, rot_base=500.0, gru_width=44,
             left_scale=0.7, right_scale=0.4, mlp="dense", ff=48)
    d.update(kw)
    return VokepelLayerSpec(**d)


def small_spec(layers=None, **kw):
    from vllm_rust_amd.vokepel import VokepelSpec
    layers = layers or [talk_layer(mlp=None), pair_layer(), talk_layer(window=0, softcap=0.0, heads=2, kv_heads=2), pair_layer(mlp=None, rot_dims=10),
                        talk_layer(heads=3, kv_heads=1, dim=9)]
    d = dict(vocab=67, width=40, layers=layers, norm_eps=1e-5, residual_mult=0.6, logit_scale=0.7, logit_softcap=11.0, loop=(1, 3, 2))
    d.update(kw)
    return VokepelSpec(**d)


def build(spec, dtype="float32", seed=0, tweak=None, block_size=4, num_blocks=96, max_tokens=320, max_seqs=6):
    from vllm_rust_amd.engine import Engine
    from vllm_rust_amd.vokepel import VokepelForCausalLM, synthetic_weights
    ck = synthetic_weights(spec, seed)
    if tweak:
        tweak(ck)
    model = VokepelForCausalLM(spec, dtype=dtype, block_size=block_size, num_blocks=num_blocks, max_tokens=max_tokens, max_seqs=max_seqs)
    model.load_state(ck)
    return model, Engine(model), {k: v.double() for k, v in ck.items()}


def rel_err(got, want):
    """Difference of two logits arrays, row means removed, relative to the spread of the expected rows (worst row)."""
    g, w = np.asarray(got, np.float64), np.asarray(want, np.float64)
    d = g - w
    d = d - d.mean(-1, keepdims=True)
    return float((np.sqrt((d ** 2).mean(-1)) / (w.std(-1) + 1e-12)).max())


def tokens_for(spec, n, seed):
    return np.random.default_rng(seed).integers(0, spec.vocab, n).tolist()


def oracle(spec, weights, toks):
    from tests import vokepel_oracle as orc
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

def _attention_op(torch, q, k, v, scale, cap, window, block_size, dtype, gate=None, sink=None, r1=None, r2=None, talk=None, gate_elem=False,
                  seed=1, runs=False, pos0=0):
    """vmx_window_attention_ex for ONE sequence whose blocks are scattered over a larger cache; the last T - pos0 positions are the
    queries (pos0 > 0: earlier rows are already cached).  runs: hand the operator seq_starts (matrix-core forms where sizes and
    cache allow); runs == "split": also a workspace, so that a run's keys are dealt to several workgroups and merged."""
    import ctypes as C
    from vllm_rust_amd._lib import WindowAttnExtras, check, lib
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
    gd = None if gate is None else gate[pos0:].float().contiguous().cuda()
    st = torch.tensor([0, n], dtype=torch.int32, device="cuda")
    ws = torch.empty(lib.vmx_window_attention_workspace_bytes(n, H, V) // 4, dtype=torch.float32, device="cuda")
    keep = [None if t is None else t.to(torch.bfloat16).cuda() for t in (sink, r1, r2, talk)]
    ex = WindowAttnExtras(*[None if t is None else t.data_ptr() for t in keep], 1 if gate_elem else 0)
    check(lib.vmx_window_attention_ex(out.data_ptr(), 0, qd.data_ptr(), H * D, kc.data_ptr(), vc.data_ptr(), dtype, bt.data_ptr(), nb, sid.data_ptr(),
                                      pid.data_ptr(), None, None if gd is None else gd.data_ptr(), 0 if gd is None else gd.shape[1], scale, cap, window,
                                      0, n, H, G, D, V, block_size, st.data_ptr() if runs else None, 1 if runs else 0,
                                      ws.data_ptr() if runs == "split" else None, ws.numel() * 4, C.byref(ex), None))
    torch.cuda.synchronize()
    return out.cpu().double().reshape(n, H, V)


FORMS = [(0, False), (1, False), (1, True), (1, "split")]   # (cache dtype, runs): f32 vector, bf16 vector, matrix cores, + key shares


def _rand_qkv(torch, T, H, G, D, V, seed, bf16):
    g = torch.Generator().manual_seed(seed)
    q, k, v = (torch.randn(s, generator=g, dtype=torch.float64) for s in ((T, H, D), (T, G, D), (T, G, V)))
    if bf16:   # the cache rounds keys and values, the matrix-core forms the queries: give them representable numbers
        q, k, v = (t.to(torch.bfloat16).double() for t in (q, k, v))
    return q, k, v, g


@pytest.mark.parametrize("form", FORMS)
@pytest.mark.parametrize("H,G,D,V,window,bs", [(4, 2, 16, 24, 9, 4), (6, 2, 8, 8, 0, 16), (3, 1, 11, 11, 5, 3), (8, 8, 64, 64, 40, 16), (12, 2, 32, 32, 70, 8),
                                              (1, 1, 40, 16, 1, 1), (16, 2, 128, 128, 100, 16)])
@pytest.mark.parametrize("kind", ["sink", "talk"])
def test_attention_extras(gpu, form, H, G, D, V, window, bs, kind):
    _, torch = gpu
    from tests import vokepel_oracle as orc
    dtype, runs = form
    T = 150
    if kind == "talk":
        V = D
    q, k, v, g = _rand_qkv(torch, T, H, G, D, V, 5 + H, dtype == 1)
    bfr = lambda t: t.to(torch.bfloat16).double()
    if kind == "sink":
        sink = bfr(torch.randn(H, generator=g, dtype=torch.float64) * 2)
        want = orc.windowed_attention(q, k, v, 0.3, window, sink=sink)
        got = _attention_op(torch, q, k, v, 0.3, 0.0, window, bs, dtype, sink=sink, runs=runs)
    else:
        r1, r2 = bfr(torch.rand(H, generator=g, dtype=torch.float64)), bfr(torch.rand(H, generator=g, dtype=torch.float64) + 0.1)
        talk = bfr(torch.eye(H, dtype=torch.float64) + 0.3 * torch.randn(H, H, generator=g, dtype=torch.float64))
        gate = torch.randn(T, H * V, generator=g, dtype=torch.float64)
        want = orc.windowed_attention(q, k, v, 0.3, window, 6.0, r1, r2, talk) * torch.sigmoid(gate).reshape(T, H, V)
        got = _attention_op(torch, q, k, v, 0.3, 6.0, window, bs, dtype, gate=gate, r1=r1, r2=r2, talk=talk, gate_elem=True, runs=runs)
    tol = 2e-5 if dtype == 0 else 6e-3
    assert float((got - want).abs().max()) < tol * max(1.0, float(want.abs().max()))


@pytest.mark.parametrize("form", FORMS)
@pytest.mark.parametrize("kind", ["sink", "talk"])
@pytest.mark.parametrize("window,bs", [(40, 16), (64, 16), (65, 8), (17, 5), (128, 16)])
def test_attention_needle_at_the_window_edge(gpu, form, kind, window, bs):
    """One key carries a score far above the rest.  Queries at distance window - 1 (the last that see it) and window (the first
    that do not), in a prompt and as single decoded rows, on several page sizes; a far key among hundreds without a window."""
    _, torch = gpu
    from tests import vokepel_oracle as orc
    dtype, runs = form
    H, G, D = 4, 2, 16
    T = 330
    q, k, v, g = _rand_qkv(torch, T, H, G, D, D, 3, dtype == 1)
    q, k = q * 0.2, k * 0.2
    needle = 37
    d = torch.randn(G, D, generator=g, dtype=torch.float64).sign()
    k[needle] = d                                     # score 16 against a query along d; every other score is of order 1
    for i in (needle + window - 1, needle + window):
        q[i] = d.repeat_interleave(H // G, dim=0)
    bfr = lambda t: t.to(torch.bfloat16).double()
    q, k = bfr(q), bfr(k)
    kw = dict(sink=bfr(torch.randn(H, generator=g, dtype=torch.float64))) if kind == "sink" else \
        dict(r1=bfr(torch.full((H,), 0.05, dtype=torch.float64)), r2=bfr(torch.full((H,), 0.5, dtype=torch.float64)),
             talk=bfr(torch.eye(H, dtype=torch.float64) + 0.1 * torch.randn(H, H, generator=g, dtype=torch.float64)))
    tol = 2e-5 if dtype == 0 else 8e-3
    for win in (window, 0):   # 0: no window, the needle stays visible from 292 keys away
        want = orc.windowed_attention(q, k, v, 1.0, win, **kw)
        got = _attention_op(torch, q, k, v, 1.0, 0.0, win, bs, dtype, runs=runs, **kw)
        assert float((got - want).abs().max()) < tol * max(1.0, float(want.abs().max()))
        # the needle decides the row just inside, and is gone just outside
        inside, outside = want[needle + window - 1], want[needle + window]
        assert float((inside - v[needle].repeat_interleave(H // G, dim=0)).abs().max()) < 0.2 or kind == "talk"
        if win:
            assert float((outside - v[needle].repeat_interleave(H // G, dim=0)).abs().max()) > 0.2
        for i in (needle + window - 1, needle + window, T - 1):   # the same rows decoded alone over the cached keys
            one = _attention_op(torch, q[:i + 1], k[:i + 1], v[:i + 1], 1.0, 0.0, win, bs, dtype, runs=runs, pos0=i, **kw)
            assert float((one[0] - want[i]).abs().max()) < tol * max(1.0, float(want.abs().max()))


@pytest.mark.parametrize("qw,kw_,hd,rot,norms", [(48, 24, 12, 8, False), (48, 24, 12, 0, True), (30, 10, 10, 10, True), (256, 128, 64, 64, False),
                                                (7, 7, 7, 0, True), (1536, 512, 128, 32, True)])
@pytest.mark.parametrize("dtype", [0, 1])
def test_qk_prepare(gpu, qw, kw_, hd, rot, norms, dtype):
    _, torch = gpu
    from tests import vokepel_oracle as orc
    from vllm_rust_amd._lib import check, lib
    T, vw, base, eps = 9, 20, 777.0, 1e-5
    g = torch.Generator().manual_seed(qw)
    q, k, v = (torch.randn(T, n, generator=g, dtype=torch.float64) for n in (qw, kw_, vw))
    qn, kn = (1 + 0.2 * torch.randn(n, generator=g, dtype=torch.float64) for n in (qw, kw_))
    qn, kn = qn.to(torch.bfloat16), kn.to(torch.bfloat16)
    pos = torch.tensor([0, 1, 2, 3, 50, 51, 1000, 1001, 5000], dtype=torch.int32)
    slots = torch.tensor([5, 4, -1, 0, 1, 2, 11, 10, 7], dtype=torch.int32)
    fused = torch.cat([q, k, v], 1).float().cuda()
    ld = qw + kw_ + vw
    qo = torch.empty(T, qw, dtype=torch.float32, device="cuda")
    cdt = torch.float32 if dtype == 0 else torch.bfloat16
    kc, vc = torch.zeros(12, kw_, dtype=cdt, device="cuda"), torch.zeros(12, vw, dtype=cdt, device="cuda")
    inv = torch.tensor([base ** (-2.0 * i / rot) for i in range(rot // 2)], dtype=torch.float32, device="cuda") if rot else None
    qnd, knd, posd, slotsd = qn.cuda(), kn.cuda(), pos.cuda(), slots.cuda()
    check(lib.vmx_qk_prepare_cache_write(qo.data_ptr(), fused.data_ptr(), ld, qw, fused.data_ptr() + 4 * qw, ld, kw_, fused.data_ptr() + 4 * (qw + kw_), ld,
                                         vw, qnd.data_ptr() if norms else None, knd.data_ptr() if norms else None, eps,
                                         None if inv is None else inv.data_ptr(), rot, hd, posd.data_ptr(), slotsd.data_ptr(),
                                         kc.data_ptr(), vc.data_ptr(), dtype, T, None))
    torch.cuda.synchronize()
    qf, kf = q.float().double(), k.float().double()
    if norms:
        qf, kf = orc.rms_norm(qf, qn.double(), eps), orc.rms_norm(kf, kn.double(), eps)
    if rot:
        qf = torch.stack([orc.rotate_pairs(qf[t].reshape(-1, hd), int(pos[t]), rot, base).reshape(-1) for t in range(T)])
        kf = torch.stack([orc.rotate_pairs(kf[t].reshape(-1, hd), int(pos[t]), rot, base).reshape(-1) for t in range(T)])
    # angles are f32 products of a position and an f32 step: at position 5000 they carry an error of about 5000 * 2^-24
    tol = 1e-5 if not rot else 6e-3
    assert float((qo.cpu().double() - qf).abs().max()) < tol * 4
    for t in range(T):
        s = int(slots[t])
        if s >= 0:
            assert float((kc[s].cpu().double() - kf[t]).abs().max()) < (tol * 4 if dtype == 0 else 0.04)
            assert float((vc[s].cpu().double() - v[t].float().double()).abs().max()) < (1e-6 if dtype == 0 else 0.04)
    assert float(kc[3].abs().max()) == 0 and float(kc[6].abs().max()) == 0   # untouched rows (slot -1 wrote nothing)


@pytest.mark.parametrize("width", [1, 44, 64, 200])
def test_min_gru_in_portions_through_dirty_slots(gpu, width):
    """Three sequences of unequal length fed in unequal portions (1 .. 90 rows a step, so strands of 1 .. 6 rows) through slots that
    start full of NaN; outputs against the oracle's recurrence over the whole sequences."""
    _, torch = gpu
    from tests import vokepel_oracle as orc
    from vllm_rust_amd._lib import check, lib
    g = torch.Generator().manual_seed(width)
    lens = [131, 1, 47]
    zl, u, gt = ([torch.randn(n, width, generator=g, dtype=torch.float64).float() * 2 for n in lens] for _ in range(3))
    state = torch.full((5, width), float("nan"), dtype=torch.float32, device="cuda")
    slot_of = [3, 0, 4]
    got = [[] for _ in lens]
    fed = [0, 0, 0]
    portions = [[90, 1, 1, 37, 2], [1], [2, 3, 40, 1, 1]]
    for step in range(5):
        rows, starts, slots, posn, owners = [], [0], [], [], []
        for s, n in enumerate(lens):
            if step < len(portions[s]) and fed[s] < n:
                c = min(portions[s][step], n - fed[s])
                rows.append(torch.cat([zl[s][fed[s]:fed[s] + c], u[s][fed[s]:fed[s] + c], gt[s][fed[s]:fed[s] + c]], 1))
                posn += list(range(fed[s], fed[s] + c))
                starts.append(starts[-1] + c)
                slots.append(slot_of[s])
                owners.append((s, c))
                fed[s] += c
        x = torch.cat(rows).cuda()
        T = x.shape[0]
        y = torch.empty(T, width, dtype=torch.float32, device="cuda")
        i32 = lambda a: torch.tensor(a, dtype=torch.int32, device="cuda")
        P, S, L = i32(posn), i32(starts), i32(slots)
        check(lib.vmx_min_gru(y.data_ptr(), 0, x.data_ptr(), 3 * width, x.data_ptr() + 4 * width, 3 * width, x.data_ptr() + 8 * width, 3 * width,
                              state.data_ptr(), P.data_ptr(), S.data_ptr(), L.data_ptr(), len(slots), T, width, None))
        torch.cuda.synchronize()
        at = 0
        for s, c in owners:
            got[s].append(y[at:at + c].cpu())
            at += c
    for s, n in enumerate(lens):
        want = orc.min_gru_states(zl[s].double(), u[s].double()) * orc.silu(gt[s].double())
        assert fed[s] == n
        assert float((torch.cat(got[s]).double() - want).abs().max()) < 2e-5


# ----------------------------------------------------------------------------- the executor through the engine

@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_layers_and_logits_against_the_oracle(gpu, dtype):
    spec = small_spec()
    model, eng, w = build(spec, dtype)
    toks = tokens_for(spec, 41, 1)
    lg, _, tr = eng.step([("a", toks, list(range(len(toks))))], layer_trace=True)
    want, wtr = oracle(spec, w, toks)
    assert tr.shape[0] == len(spec.layer_runs) == 7
    for r in range(tr.shape[0]):
        assert rel_err(tr[r].cpu().numpy(), wtr[r]) < TOL[dtype], f"layer run {r}"
    assert rel_err(lg.cpu().numpy(), want) < TOL[dtype]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_prompt_decode_and_portions_agree(gpu, dtype):
    spec = small_spec()
    model, eng, w = build(spec, dtype)
    toks = tokens_for(spec, 53, 2)
    want, _ = oracle(spec, w, toks)
    for cuts in ([53], [1], [2], [3], [7, 16], [16, 1], [20, 2, 1]):
        got = feed(eng, "s", toks, cuts)
        assert rel_err(got, want) < TOL[dtype], f"cuts {cuts}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_unequal_batches_and_recycled_blocks_and_slots(gpu, dtype):
    """Four requests of unequal length in one batch, then decoded together while the short ones finish early; five generations of
    requests through 3 state slots and few blocks, freed blocks and slots handed out again in another order."""
    spec = small_spec()
    model, eng, w = build(spec, dtype, num_blocks=40, max_seqs=3)
    for gen in range(5):
        lens = [(29, 6), (3, 2), (14, 9)]
        reqs = {f"g{gen}r{i}": tokens_for(spec, n + d, 100 * gen + i) for i, (n, d) in enumerate(lens)}
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
    spec = small_spec(layers=[talk_layer(window=window), pair_layer(window=window), talk_layer(window=window + 1, mlp=None)], loop=(0, 2, 2))
    model, eng, w = build(spec, dtype, block_size=bs, num_blocks=max(24, 400 // bs))
    toks = tokens_for(spec, 45, window)
    want, _ = oracle(spec, w, toks)
    assert rel_err(feed(eng, "a", toks, [45]), want) < TOL[dtype]
    assert rel_err(feed(eng, "b", toks, [20, 1]), want) < TOL[dtype]
    assert rel_err(feed(eng, "c", toks, [5, 2]), want) < TOL[dtype]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("sizes", ["any", "eights"])
def test_sharp_attention_over_300_tokens_and_long_decoding(gpu, dtype, sizes):
    """Scores scaled up so that single keys decide rows, windows of 70 / 130 keys over page borders, 220 tokens as a prompt and
    80 decoded one by one; the state of the recurrent unit is carried through all of them."""
    def sharpen(ck):
        for k in ck:
            if k.endswith("mix.q") or k.endswith("left.q"):
                ck[k] = (ck[k].float() * 3).to(ck[k].dtype)
    if sizes == "any":
        layers = [pair_layer(window=70), talk_layer(window=130, scale=1.5), pair_layer(window=0, mlp=None)]
    else:    # multiples of 8: the matrix-core forms in bfloat16, windows over several key tiles
        layers = [pair_layer(window=70, dim=16, vdim=24, rot_dims=8), talk_layer(window=130, scale=1.5, dim=16),
                  pair_layer(window=0, mlp=None, dim=32, vdim=8, rot_dims=32)]
    spec = small_spec(layers=layers, loop=(0, 2, 2))
    model, eng, w = build(spec, dtype, tweak=sharpen, block_size=16, num_blocks=64, max_tokens=512)
    toks = tokens_for(spec, 300, 9)
    want, _ = oracle(spec, w, toks)
    assert rel_err(feed(eng, "a", toks, [220, 1]), want) < TOL[dtype]
    assert rel_err(feed(eng, "b", toks, [300]), want) < TOL[dtype]


OTHER_SIZES = {
    "no loop": dict(loop=None),
    "loop of one pass over everything": dict(loop=(0, 5, 1)),
    "loop at the end": dict(loop=(3, 5, 3)),
    "one layer looped": dict(layers=[pair_layer()], loop=(0, 1, 4)),
    "no caps, unit multipliers": dict(logit_softcap=0.0, logit_scale=1.0, residual_mult=1.0),
    "one head": dict(layers=[talk_layer(heads=1, kv_heads=1), pair_layer(heads=1, kv_heads=1)], loop=(0, 1, 2)),
    "equal head counts": dict(layers=[talk_layer(heads=4, kv_heads=4), pair_layer(heads=4, kv_heads=4)], loop=None),
    "many heads per key head": dict(layers=[talk_layer(heads=10, kv_heads=2, dim=8), pair_layer(heads=12, kv_heads=2, dim=8, vdim=8, rot_dims=8)], loop=(1, 2, 2)),
    "nine waves of heads": dict(layers=[talk_layer(heads=18, kv_heads=3, dim=8), pair_layer()], loop=None),
    "sizes of 8s": dict(layers=[talk_layer(heads=8, kv_heads=2, dim=32, window=40), pair_layer(heads=8, kv_heads=4, dim=64, vdim=32, rot_dims=32, gru_width=96)],
                        width=64, loop=(0, 2, 2)),
    "odd sizes": dict(layers=[talk_layer(heads=3, kv_heads=3, dim=7), pair_layer(heads=2, kv_heads=1, dim=6, vdim=5, rot_dims=2, gru_width=1)], width=34,
                      loop=(0, 1, 2)),
    "no rotation, no window": dict(layers=[pair_layer(rot_dims=0, window=0), talk_layer(window=0)], loop=None),
    "wide values": dict(layers=[pair_layer(dim=16, vdim=136, rot_dims=16), talk_layer(dim=72)], loop=None),
    "key size 130": dict(layers=[pair_layer(dim=130, vdim=8, rot_dims=64), talk_layer(heads=2, kv_heads=1, dim=132)], loop=None),
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(OTHER_SIZES))
def test_other_sizes(gpu, dtype, name):
    spec = small_spec(**OTHER_SIZES[name])
    model, eng, w = build(spec, dtype)
    toks = tokens_for(spec, 37, 4)
    want, wtr = oracle(spec, w, toks)
    lg, _, tr = eng.step([("a", toks, list(range(37)))], layer_trace=True)
    assert tr.shape[0] == len(spec.layer_runs)
    assert rel_err(tr[-1].cpu().numpy(), wtr[-1]) < TOL[dtype]
    assert rel_err(lg.cpu().numpy(), want) < TOL[dtype]
    eng.finish("a")
    assert rel_err(feed(eng, "b", toks, [30, 1]), want) < TOL[dtype]
    assert rel_err(feed(eng, "c", toks, [2]), want) < TOL[dtype]


def random_spec(rng):
    layers = []
    for _ in range(int(rng.integers(1, 6))):
        G = int(rng.integers(1, 4))
        H = G * int(rng.integers(1, 7))
        mult8 = rng.random() < 0.5
        D = int(rng.integers(1, 6)) * 8 if mult8 else 2 * int(rng.integers(2, 30))
        window = int(rng.choice([0, 1, 2, 5, 16, 33, 64]))
        mlp = "dense" if rng.random() < 0.7 else None
        ff = int(rng.integers(8, 90))
        if rng.random() < 0.5:
            layers.append(talk_layer(heads=H, kv_heads=G, dim=D, window=window, scale=float(rng.uniform(0.1, 0.6)),
                                     softcap=float(rng.choice([0.0, 4.0, 30.0])), mlp=mlp, ff=ff))
        else:
            V = int(rng.integers(1, 6)) * 8 if mult8 else int(rng.integers(3, 70))
            layers.append(pair_layer(heads=H, kv_heads=G, dim=D, vdim=V, window=window, scale=float(rng.uniform(0.1, 0.6)),
                                     rot_dims=2 * int(rng.integers(0, D // 2 + 1)), rot_base=float(rng.choice([100.0, 1e4, 1e6])),
                                     gru_width=int(rng.integers(1, 150)), left_scale=float(rng.uniform(0.3, 1.2)),
                                     right_scale=float(rng.uniform(0.3, 1.2)), mlp=mlp, ff=ff))
    n = len(layers)
    loop = None
    if rng.random() < 0.7:
        a = int(rng.integers(0, n))
        loop = (a, int(rng.integers(a + 1, n + 1)), int(rng.integers(1, 4)))
    return small_spec(layers=layers, width=int(rng.integers(3, 12)) * 8 if rng.random() < 0.5 else int(rng.integers(9, 90)), vocab=int(rng.integers(20, 300)),
                      residual_mult=float(rng.uniform(0.3, 1.0)), logit_scale=float(rng.uniform(0.3, 1.5)),
                      logit_softcap=float(rng.choice([0.0, 8.0, 30.0])), loop=loop, norm_eps=float(rng.choice([1e-6, 1e-5])))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", range(12))
def test_random_models(gpu, dtype, seed):
    """Models drawn at random (layer order, loops, head counts, sizes, windows, caps, rotations) on random page sizes: two unequal
    requests decoding together, a third fed in portions."""
    rng = np.random.default_rng(seed)
    spec = random_spec(rng)
    bs = int(rng.choice([1, 3, 4, 8, 16]))
    model, eng, w = build(spec, dtype, seed=seed, block_size=bs, num_blocks=600 // bs + 8)
    ta, tb, tc = tokens_for(spec, 75, seed), tokens_for(spec, 33, seed + 50), tokens_for(spec, 60, seed + 99)
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
            lg, _ = oracle(spec, w, seq)
            top2 = np.sort(lg[-1])[-2:]
            if top2[1] - top2[0] > 1e-3:      # a tie within rounding says nothing
                assert int(np.argmax(lg[-1])) == t
            seq.append(t)
    assert len(eng.blocks.free) == 30 and len(eng.states.free) == 3
    outs = eng.generate(prompts[:3], SamplingParams(temperature=0.9, top_k=20, top_p=0.9, max_new_tokens=5, seed=3))
    assert all(len(o) == 5 and all(0 <= t < spec.vocab for t in o) for o in outs)


def torch_ones(n):
    import torch
    return torch.ones(n, dtype=torch.bfloat16)


def _write_checkpoint(tmp_path, spec, seed=0):
    from safetensors.torch import save_file
    from vllm_rust_amd.vokepel import synthetic_weights
    ck = synthetic_weights(spec, seed)
    d = tmp_path / "model"
    d.mkdir()
    (d / "config.json").write_text(json.dumps(spec.to_config()))
    extra = {f"l{i}.norm2": torch_ones(spec.width) for i, l in enumerate(spec.layers) if l.mlp is None}   # a file may carry them: skipped
    save_file({k: v.contiguous() for k, v in {**ck, **extra}.items()}, str(d / "model.safetensors"))
    return d, {k: v.double() for k, v in ck.items()}


def test_registry_and_command_line_tools(gpu, tmp_path):
    """A checkpoint directory written here: the registry picks the class from config.json; bin/trace_run replays a trace (a prompt,
    a portion, decode steps of two requests, an early finisher) in both modes; bin/generate continues greedily."""
    from vllm_rust_amd.engine import Engine
    from vllm_rust_amd.models import architecture_of, load_model
    spec = small_spec()
    d, w = _write_checkpoint(tmp_path, spec)
    assert architecture_of(d) == "Vokepel"
    model = load_model(d, dtype="float32", max_tokens=128, max_seqs=4, block_size=8)
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

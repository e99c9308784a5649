"""Host-side driver of the Gezozen decoder family (libvmx `vmx_gezozen_*`).

A Gezozen model is a stack of layers listed in its config.json that normalise after the sum, `x <- N1(a x + gate1 * mixer(x));
x <- N2(a x + gate2 * ff(x))`, with sigmoid gates computed from the sublayer's input, one constant `a` for the model and a
root-mean-square norm N taken over equal consecutive groups of the row.  Mixers: "parallel" (grouped-query attention with
per-head q/k norms, rotation in halves and soft-capped scores beside gated linear attention), "parallel_2" (the same attention
with biased projections, stretched rotation frequencies and a sliding window beside retention) and "delta" (short convolutions
and the gated delta rule with one decay per head).  Feed-forward: "moe", sigmoid-routed gated experts whose routing score scales
the expert's input, plus a gated shared expert.  This file reads the configuration, hands the checkpoint's tensors to the
library under their file names and wraps the one forward entry point.  All arithmetic happens in the library.
"""
from __future__ import annotations

import ctypes as C
import dataclasses
import json
import math
import re
from pathlib import Path

import numpy as np
import torch

from ._lib import GezozenConfig, GezozenLayerConfig, Rotation, check, lib

VMX_F32, VMX_BF16 = 0, 1
MIXERS = {"parallel": 5, "parallel_2": 6, "delta": 7}
MLPS = {None: 0, "moe": 5}


@dataclasses.dataclass
class RotationSpec:
    dims: int = 0                # rotated coordinates per head (0: none)
    base: float = 10000.0
    scaling: dict | None = None  # {factor, original, fast, slow}: slow pairs turn `factor` times slower

    @staticmethod
    def from_config(rot: dict | None) -> "RotationSpec":
        if not rot or not rot.get("dims"):
            return RotationSpec()
        sc = rot.get("scaling")
        return RotationSpec(int(rot["dims"]), float(rot["base"]),
                            {k: float(sc[k]) for k in ("factor", "original", "fast", "slow")} if sc else None)

    def to_config(self) -> dict | None:
        if not self.dims:
            return None
        d = {"base": self.base, "dims": self.dims}
        if self.scaling:
            d["scaling"] = dict(self.scaling)
        return d

    def to_struct(self) -> Rotation:
        sc = self.scaling or {}
        return Rotation(self.dims, self.base, sc.get("factor", 0.0), sc.get("original", 0.0), sc.get("fast", 0.0), sc.get("slow", 0.0))


@dataclasses.dataclass
class GezozenLayerSpec:
    mixer: str = "delta"
    # attention of the two-sided mixers / heads of the delta rule (heads: value heads, kv_heads: query and key heads)
    heads: int = 4
    kv_heads: int = 2
    dim: int = 32
    vdim: int = 32
    window: int = 0              # 0: every earlier key
    scale: float = 0.125
    softcap: float = 0.0         # 0: none
    rot: RotationSpec = dataclasses.field(default_factory=RotationSpec)
    # recurrent right side of the two-sided mixers
    r_heads: int = 0
    r_dim: int = 0
    r_vdim: int = 0
    tau: float = 1.0             # parallel: decay = sigmoid(z)^(1 / tau)
    decay_rank: int = 0          # parallel: inner size of the decay projection
    decay: tuple = ()            # parallel_2: one constant decay per head
    r_rot: RotationSpec = dataclasses.field(default_factory=RotationSpec)
    left_scale: float = 1.0
    right_scale: float = 1.0
    conv: int = 4                # delta: taps of the short convolutions
    mlp: str | None = "moe"
    experts: int = 4
    top: int = 1
    expert_ff: int = 32
    shared_ff: int = 0           # 0: no shared expert

    @property
    def qkv_bias(self) -> bool:
        return self.mixer == "parallel_2"

    @staticmethod
    def from_config(entry: dict, decay_rank: int = 0) -> "GezozenLayerSpec":
        """decay_rank: inner size of the gated linear attention's decay projection; the configuration does not list it (the
        checkpoint's tensor shape does)."""
        kind = entry["type"]
        if kind not in MIXERS:
            raise ValueError(f"Gezozen: unknown layer type `{kind}`")
        m = entry["mixer"]
        s = GezozenLayerSpec(mixer=kind, mlp=None)
        if kind == "delta":
            s.heads, s.kv_heads, s.dim, s.vdim = int(m["heads"]), int(m.get("kv_heads", m["heads"])), int(m["dim"]), int(m.get("vdim", m["dim"]))
            s.conv = int(m["conv"])
        else:
            a, r = m["left"], m["right"]
            s.heads, s.kv_heads, s.dim, s.vdim = int(a["heads"]), int(a.get("kv_heads", a["heads"])), int(a["dim"]), int(a.get("vdim", a["dim"]))
            s.window = int((a.get("mask") or {}).get("size") or 0)
            s.scale = float(a.get("scale", 1.0 / math.sqrt(s.dim)))
            s.softcap = float(a.get("softcap") or 0.0)
            s.rot = RotationSpec.from_config(a.get("rot"))
            s.r_heads, s.r_dim, s.r_vdim = int(r["heads"]), int(r["dim"]), int(r.get("vdim", r["dim"]))
            s.left_scale, s.right_scale = float(m.get("left_scale", 1.0)), float(m.get("right_scale", 1.0))
            if kind == "parallel":
                s.tau, s.decay_rank = float(r["tau"]), int(decay_rank)
            else:
                s.decay = tuple(float(d) for d in r["decay"])
                if len(s.decay) != s.r_heads:
                    raise ValueError(f"Gezozen: {len(s.decay)} decays for {s.r_heads} retention heads")
                s.r_rot = RotationSpec.from_config(r.get("rot"))
        ff = entry.get("mlp")
        if ff is not None:
            if ff["kind"] != "moe":
                raise ValueError(f"Gezozen: unknown feed-forward kind `{ff['kind']}`")
            s.mlp, s.experts, s.top = "moe", int(ff["router"]["experts"]), int(ff["router"]["top"])
            s.expert_ff = int(ff["expert"]["ff"])
            s.shared_ff = int((ff.get("shared") or {}).get("ff") or 0)
        return s

    def to_config(self) -> dict:
        if self.mixer == "delta":
            m = {"conv": self.conv, "dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "vdim": self.vdim}
        else:
            a = {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "vdim": self.vdim, "scale": self.scale}
            if self.window:
                a["mask"] = {"size": self.window}
            if self.softcap:
                a["softcap"] = self.softcap
            if self.rot.dims:
                a["rot"] = self.rot.to_config()
            r = {"dim": self.r_dim, "heads": self.r_heads, "vdim": self.r_vdim}
            if self.mixer == "parallel":
                r["tau"] = self.tau
            else:
                r["decay"] = list(self.decay)
                if self.r_rot.dims:
                    r["rot"] = self.r_rot.to_config()
            m = {"left": a, "right": r, "left_scale": self.left_scale, "right_scale": self.right_scale}
        ff = None
        if self.mlp:
            ff = {"kind": "moe", "expert": {"ff": self.expert_ff}, "router": {"experts": self.experts, "top": self.top}}
            if self.shared_ff:
                ff["shared"] = {"ff": self.shared_ff}
        return {"type": self.mixer, "mixer": m, "mlp": ff}


@dataclasses.dataclass
class GezozenSpec:
    vocab: int
    width: int
    layers: list
    norm_eps: float = 1e-6
    norm_groups: int = 1
    postln_alpha: float = 1.0

    @staticmethod
    def from_config(cfg: dict, decay_ranks: dict | None = None) -> "GezozenSpec":
        """decay_ranks: {layer index: inner size of that layer's decay projection}, read off the checkpoint's tensor shapes."""
        ranks = decay_ranks or {}
        return GezozenSpec(vocab=int(cfg["vocab"]), width=int(cfg["width"]),
                           layers=[GezozenLayerSpec.from_config(e, ranks.get(i, 0)) for i, e in enumerate(cfg["layers"])],
                           norm_eps=float(cfg["norm"]["eps"]), norm_groups=int(cfg["norm"].get("groups", 1)),
                           postln_alpha=float(cfg.get("postln_alpha", 1.0)))

    def to_config(self) -> dict:
        return {"architecture": "Gezozen", "vocab": self.vocab, "width": self.width, "norm": {"eps": self.norm_eps, "groups": self.norm_groups},
                "postln_alpha": self.postln_alpha, "layers": [l.to_config() for l in self.layers]}

    def tensor_shapes(self) -> dict:
        """Name -> shape of every checkpoint tensor, in file order."""
        W, out = self.width, {}
        out["embed"] = (self.vocab, W)
        for i, l in enumerate(self.layers):
            p = f"l{i}."
            out[p + "norm1"] = (W,)
            if l.mlp:
                out[p + "norm2"] = (W,)
            H, G, D, V = l.heads, l.kv_heads, l.dim, l.vdim
            if l.mixer == "delta":
                n = l.conv
                out[p + "mix.q"], out[p + "mix.q.conv"] = (G * D, W), (G * D, n)
                out[p + "mix.k"], out[p + "mix.k.conv"] = (G * D, W), (G * D, n)
                out[p + "mix.v"], out[p + "mix.v.conv"] = (H * V, W), (H * V, n)
                out[p + "mix.b"], out[p + "mix.A_log"], out[p + "mix.norm"] = (H, W), (H,), (V,)
                out[p + "mix.a"], out[p + "mix.dt_bias"] = (H, W), (H,)
                out[p + "mix.g"], out[p + "mix.o"] = (H * V, W), (W, H * V)
            else:
                for nm, rows in (("q", H * D), ("k", G * D), ("v", G * V)):
                    out[p + "mix.left." + nm] = (rows, W)
                    if l.qkv_bias:
                        out[p + "mix.left." + nm + ".b"] = (rows,)
                out[p + "mix.left.q.norm"], out[p + "mix.left.k.norm"] = (D,), (D,)
                out[p + "mix.left.o"] = (W, H * V)
                RH, RD, RV = l.r_heads, l.r_dim, l.r_vdim
                out[p + "mix.right.q"], out[p + "mix.right.k"] = (RH * RD, W), (RH * RD, W)
                out[p + "mix.right.v"], out[p + "mix.right.g"], out[p + "mix.right.o"] = (RH * RV, W), (RH * RV, W), (W, RH * RV)
                if l.mixer == "parallel":
                    out[p + "mix.right.norm"] = (RV,)
                    out[p + "mix.right.a1"], out[p + "mix.right.a2"], out[p + "mix.right.a2.b"] = (l.decay_rank, W), (RH * RD, l.decay_rank), (RH * RD,)
            if l.mlp:
                for e in range(l.experts):
                    out[p + f"mlp.e{e}.gate"], out[p + f"mlp.e{e}.up"], out[p + f"mlp.e{e}.down"] = (l.expert_ff, W), (l.expert_ff, W), (W, l.expert_ff)
                out[p + "mlp.router"] = (l.experts, W)
                if l.shared_ff:
                    out[p + "mlp.shared.gate"], out[p + "mlp.shared.up"] = (l.shared_ff, W), (l.shared_ff, W)
                    out[p + "mlp.shared.down"], out[p + "mlp.shared.sg"] = (W, l.shared_ff), (1, W)
            out[p + "rg1"], out[p + "rg1.b"] = (W, W), (W,)
            if l.mlp:
                out[p + "rg2"], out[p + "rg2.b"] = (W, W), (W,)
        out["final.norm"] = (W,)
        out["head"] = (self.vocab, W)
        return out


def synthetic_weights(spec: GezozenSpec, seed: int = 0, device="cpu") -> dict:
    """Seeded random-init checkpoint (bf16 tensors on `device`): matrices ~ 1 / sqrt(in), gains around 1, biases of order 1,
    decay constants that keep the memories' time scales between a few and a few hundred tokens."""
    g = torch.Generator(device=device).manual_seed(seed)

    def randn(shape):
        return torch.randn(shape, generator=g, device=device)
    ck = {}
    for name, shape in spec.tensor_shapes().items():
        if name.endswith("norm1") or name.endswith("norm2") or name.endswith(".norm"):
            t = 1.0 + 0.1 * randn(shape)
        elif name.endswith(".conv"):
            t = 0.5 * randn(shape)
        elif name.endswith("A_log"):
            t = -1.0 + 0.5 * randn(shape)
        elif name.endswith("dt_bias"):
            t = -1.0 + randn(shape)
        elif name.endswith("a2.b"):
            t = 3.0 + randn(shape)
        elif name.endswith(".b") and len(shape) == 1:
            t = 0.5 * randn(shape)
        elif name == "embed":
            t = randn(shape)
        else:
            t = randn(shape) / math.sqrt(shape[-1])
        ck[name] = t.to(torch.bfloat16)
    return ck


class GezozenForCausalLM:
    """The executor handle: weights, paged key/value caches, recurrent-state slots and workspaces live in the library."""

    architecture = "Gezozen"

    def __init__(self, spec: GezozenSpec, dtype: str = "bfloat16", block_size: int = 16, num_blocks: int = 256, max_tokens: int = 2048,
                 max_seqs: int = 64, device: int = 0):
        if dtype not in ("bfloat16", "float32"):
            raise ValueError(f"Gezozen runs in bfloat16 or float32, not `{dtype}`")
        self.spec, self.dtype = spec, dtype
        self.block_size, self.num_blocks, self.max_tokens, self.max_seqs = block_size, num_blocks, max_tokens, max_seqs
        self.vocab_size = spec.vocab
        self.state_slots = max_seqs          # the engine hands one to every live sequence
        self.device = torch.device("cuda", device)
        cfg = GezozenConfig(spec.vocab, spec.width, len(spec.layers), spec.norm_eps, spec.norm_groups, spec.postln_alpha,
                            VMX_F32 if dtype == "float32" else VMX_BF16, block_size, num_blocks, max_tokens, max_seqs, self.state_slots)
        layers = (GezozenLayerConfig * len(spec.layers))()
        keep = []                            # host arrays the library reads during create
        for i, l in enumerate(spec.layers):
            decay = (C.c_float * max(len(l.decay), 1))(*l.decay)
            keep.append(decay)
            layers[i] = GezozenLayerConfig(MIXERS[l.mixer], l.heads, l.kv_heads, l.dim, l.vdim, l.window, l.scale, l.softcap, 1 if l.qkv_bias else 0,
                                           l.rot.to_struct(), l.r_heads, l.r_dim, l.r_vdim, l.tau, l.decay_rank,
                                           C.cast(decay, C.POINTER(C.c_float)) if l.decay else None, l.r_rot.to_struct(), l.left_scale,
                                           l.right_scale, l.conv, MLPS[l.mlp], l.experts, l.top, l.expert_ff, l.shared_ff)
        self._h = C.c_void_p()
        check(lib.vmx_gezozen_create(C.byref(cfg), layers, C.byref(self._h)))

    @classmethod
    def from_pretrained(cls, model_dir, dtype: str = "bfloat16", **kw) -> "GezozenForCausalLM":
        from .checkpoint import CheckpointDir
        cfg = json.loads((Path(model_dir) / "config.json").read_text())
        ck = CheckpointDir(model_dir)
        try:
            ranks = {}                       # the decay projections' inner sizes are shapes of the checkpoint, not configuration
            for name in ck.where:
                m = re.fullmatch(r"l(\d+)\.mix\.right\.a1", name)
                if m:
                    f = ck._file(ck.where[name])
                    ranks[int(m.group(1))] = int(f.info(lib.vmx_safetensors_find(f._h, name.encode()))[2][0])
        finally:
            ck.close()
        model = cls(GezozenSpec.from_config(cfg, ranks), dtype=dtype, **kw)
        model.load_checkpoint(model_dir)
        return model

    def close(self):
        if self._h:
            lib.vmx_gezozen_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @staticmethod
    def _stream():
        return torch.cuda.current_stream().cuda_stream

    def load_tensor(self, name: str, t) -> None:
        """t: bf16 torch tensor (host or device) or a numpy uint16 array of bf16 bit patterns."""
        if isinstance(t, np.ndarray):
            assert t.dtype == np.uint16, f"{name}: bf16 bit patterns expected"
            t = np.ascontiguousarray(t)
            check(lib.vmx_gezozen_load_tensor(self._h, name.encode(), t.ctypes.data, t.nbytes, self._stream()))
            return
        assert t.dtype == torch.bfloat16, f"{name}: bf16 expected, got {t.dtype}"
        t = t.contiguous()
        check(lib.vmx_gezozen_load_tensor(self._h, name.encode(), t.data_ptr(), t.numel() * 2, self._stream()))

    def load_state(self, tensors: dict) -> None:
        for name, t in tensors.items():
            self.load_tensor(name, t)
        self.check_loaded()

    def check_loaded(self) -> None:
        if lib.vmx_gezozen_missing_tensors(self._h) != 0:
            raise ValueError(lib.vmx_last_error().decode("utf-8", "replace"))

    def load_checkpoint(self, model_dir) -> None:
        """Every tensor of the directory's *.safetensors files under its own name (the library's safetensors reader)."""
        from .checkpoint import CheckpointDir
        ck = CheckpointDir(model_dir)
        try:
            for name in ck.where:
                f = ck._file(ck.where[name])
                dtype = f.info(lib.vmx_safetensors_find(f._h, name.encode()))[1]
                if dtype != "BF16":
                    raise ValueError(f"{model_dir}: tensor `{name}` is {dtype}; Gezozen checkpoints hold bf16")
                m = re.fullmatch(r"l(\d+)\.(norm2|rg2|rg2\.b)", name)
                if m and int(m.group(1)) < len(self.spec.layers) and self.spec.layers[int(m.group(1))].mlp is None:
                    continue                 # norm and gate of a feed-forward this layer does not have
                self.load_tensor(name, ck.get(name))
        finally:
            ck.close()
        self.check_loaded()

    def forward(self, tokens, prev_tokens, positions, slots, seq_ids, block_tables, logit_rows=None, want_logits: bool = True,
                want_greedy: bool = False, layer_trace: bool = False, seq_starts=None, state_slots=None):
        """One packed step; every argument an int32 CUDA tensor ([T] each, block_tables [S, max_blocks], seq_starts [S + 1],
        state_slots [S], logit_rows [n]); prev_tokens is not used by this design.
        Returns (logits f32 [n, vocab] or None, greedy ids int32 [n] or None, trace f32 [layers, T, width] or None)."""
        if seq_starts is None or state_slots is None:
            raise ValueError("Gezozen carries recurrent state: the step needs seq_starts and state_slots")
        T = tokens.numel()
        S = seq_starts.numel() - 1           # the sequences of THIS step; the block table may hold more rows
        if S < 1 or state_slots.numel() != S or block_tables.shape[0] < S:
            raise ValueError(f"Gezozen: {S} sequences by seq_starts, {state_slots.numel()} state slots, {block_tables.shape[0]} block-table rows")
        if not all(a.numel() == T for a in (positions, slots, seq_ids)):
            raise ValueError("Gezozen: tokens, positions, slots and seq_ids must have one entry per token")
        n = 0 if logit_rows is None else logit_rows.numel()
        logits = torch.empty((n, self.spec.vocab), dtype=torch.float32, device=self.device) if n else None
        ids = torch.empty(n, dtype=torch.int32, device=self.device) if (n and want_greedy) else None
        trace = torch.empty((len(self.spec.layers), T, self.spec.width), dtype=torch.float32, device=self.device) if layer_trace else None
        check(lib.vmx_gezozen_forward(self._h, tokens.data_ptr(), positions.data_ptr(), slots.data_ptr(), seq_ids.data_ptr(), T,
                                      block_tables.data_ptr(), S, block_tables.shape[1], seq_starts.data_ptr(),
                                      state_slots.data_ptr(), None if not n else logit_rows.data_ptr(), n,
                                      None if logits is None else logits.data_ptr(), None if ids is None else ids.data_ptr(),
                                      None if trace is None else trace.data_ptr(), self._stream()))
        return (logits if want_logits else None), ids, trace

"""Host-side driver of the Vokepel decoder family (libvmx `vmx_vokepel_*`).

A Vokepel model is a stack of pre-norm layers listed in its config.json, `x += m * mixer(norm1(x)); x += m * ff(norm2(x))` with
one residual multiplier m for the model.  Mixers: "attention" (grouped-query; the values are the keys as projected; q and k are
RMS-normed over their whole rows; scaled, soft-capped scores minus a logarithmic distance penalty, mixed across the heads before
the softmax over a sliding window; element-wise sigmoid output gate) and "parallel" (a rotary sliding-window attention with a
learned softmax sink beside a minimal gated recurrent unit whose state lives in a per-sequence state slot; the two are added
with weights from the configuration).  Feed-forward: "dense" with a squared ReLU.  A run of layers may loop: it runs several
times with the same weights, each pass entered through a matrix over [x | embedding output] plus a learned vector per pass, and
each pass keeps a cache and a state of its own.  The logits come from the embedding table, scaled and soft-capped.  This file
reads the configuration, hands the checkpoint's tensors to the library under their file names and wraps the one forward entry
point.  All arithmetic happens in the library.
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

from ._lib import VokepelConfig, VokepelLayerConfig, check, lib

VMX_F32, VMX_BF16 = 0, 1
MIXERS = {"attention": 3, "parallel": 4}
MLPS = {None: 0, "dense": 4}


@dataclasses.dataclass
class VokepelLayerSpec:
    mixer: str = "attention"
    heads: int = 4
    kv_heads: int = 2
    dim: int = 32
    vdim: int = 32
    window: int = 0              # 0: every earlier key
    scale: float = 0.125
    softcap: float = 0.0         # attention: 0 = none
    rot_dims: int = 0            # parallel: rotated coordinates per head of the left attention
    rot_base: float = 10000.0
    gru_width: int = 0           # parallel: channels of the recurrent unit
    left_scale: float = 1.0
    right_scale: float = 1.0
    mlp: str | None = "dense"
    ff: int = 64

    @staticmethod
    def from_config(entry: dict) -> "VokepelLayerSpec":
        kind = entry["type"]
        if kind not in MIXERS:
            raise ValueError(f"Vokepel: unknown layer type `{kind}`")
        m = entry["mixer"]
        a = m["left"] if kind == "parallel" else m
        s = VokepelLayerSpec(mixer=kind, heads=int(a["heads"]), kv_heads=int(a.get("kv_heads", a["heads"])), dim=int(a["dim"]),
                             vdim=int(a.get("vdim", a["dim"])), mlp=None)
        s.window = int((a.get("mask") or {}).get("size") or 0)
        s.scale = float(a.get("scale", 1.0 / math.sqrt(s.dim)))
        if kind == "attention":
            s.vdim = s.dim           # the values are the keys
            s.softcap = float(a.get("softcap") or 0.0)
        else:
            rot = a.get("rot") or {}
            s.rot_dims, s.rot_base = int(rot.get("dims") or 0), float(rot.get("base", 10000.0))
            s.gru_width = int(m["right"]["width"])
            s.left_scale, s.right_scale = float(m.get("left_scale", 1.0)), float(m.get("right_scale", 1.0))
        ff = entry.get("mlp")
        if ff is not None:
            if ff["kind"] != "dense":
                raise ValueError(f"Vokepel: unknown feed-forward kind `{ff['kind']}`")
            s.mlp, s.ff = "dense", int(ff["ff"])
        return s

    def to_config(self) -> dict:
        a = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale}
        if self.window:
            a["mask"] = {"size": self.window}
        if self.mixer == "attention":
            if self.softcap:
                a["softcap"] = self.softcap
            m = a
        else:
            if self.rot_dims:
                a["rot"] = {"base": self.rot_base, "dims": self.rot_dims}
            m = {"left": a, "right": {"width": self.gru_width}, "left_scale": self.left_scale, "right_scale": self.right_scale}
        return {"type": self.mixer, "mixer": m, "mlp": {"kind": "dense", "ff": self.ff} if self.mlp else None}


@dataclasses.dataclass
class VokepelSpec:
    vocab: int
    width: int
    layers: list
    norm_eps: float = 1e-6
    residual_mult: float = 1.0
    logit_scale: float = 1.0
    logit_softcap: float = 0.0   # 0: none
    loop: tuple | None = None    # (start, stop, times)

    @staticmethod
    def from_config(cfg: dict) -> "VokepelSpec":
        loop = cfg.get("loop")
        return VokepelSpec(vocab=int(cfg["vocab"]), width=int(cfg["width"]), layers=[VokepelLayerSpec.from_config(e) for e in cfg["layers"]],
                           norm_eps=float(cfg["norm"]["eps"]), residual_mult=float(cfg.get("residual_mult", 1.0)),
                           logit_scale=float(cfg.get("logit_scale", 1.0)), logit_softcap=float(cfg.get("logit_softcap") or 0.0),
                           loop=(int(loop["start"]), int(loop["stop"]), int(loop["times"])) if loop else None)

    def to_config(self) -> dict:
        cfg = {"architecture": "Vokepel", "vocab": self.vocab, "width": self.width, "norm": {"eps": self.norm_eps},
               "residual_mult": self.residual_mult, "logit_scale": self.logit_scale, "layers": [l.to_config() for l in self.layers]}
        if self.logit_softcap:
            cfg["logit_softcap"] = self.logit_softcap
        if self.loop:
            cfg["loop"] = {"start": self.loop[0], "stop": self.loop[1], "times": self.loop[2]}
        return cfg

    @property
    def layer_runs(self) -> list:
        """[(layer, pass or None)] in running order; a looped layer once per pass."""
        n = len(self.layers)
        if not self.loop:
            return [(i, None) for i in range(n)]
        a, b, times = self.loop
        return [(i, None) for i in range(a)] + [(i, t) for t in range(times) for i in range(a, b)] + [(i, None) for i in range(b, n)]

    def tensor_shapes(self) -> dict:
        """Name -> shape of every checkpoint tensor, in file order."""
        W, out = self.width, {}
        out["embed"] = (self.vocab, W)
        if self.loop:
            out["loop.in"], out["loop.step"] = (W, 2 * W), (self.loop[2], W)
        for i, l in enumerate(self.layers):
            p = f"l{i}."
            out[p + "norm1"] = (W,)
            if l.mlp:
                out[p + "norm2"] = (W,)
            if l.mixer == "attention":
                H, G, D = l.heads, l.kv_heads, l.dim
                out[p + "mix.q"], out[p + "mix.k"] = (H * D, W), (G * D, W)
                out[p + "mix.q.norm"], out[p + "mix.k.norm"] = (H * D,), (G * D,)
                out[p + "mix.r1"], out[p + "mix.r2"], out[p + "mix.talk"] = (H,), (H,), (H, H)
                out[p + "mix.g"], out[p + "mix.o"] = (H * D, W), (W, H * D)
            else:
                H, G, D, V, R = l.heads, l.kv_heads, l.dim, l.vdim, l.gru_width
                out[p + "mix.left.q"], out[p + "mix.left.k"], out[p + "mix.left.v"] = (H * D, W), (G * D, W), (G * V, W)
                out[p + "mix.left.sink"], out[p + "mix.left.o"] = (H,), (W, H * V)
                out[p + "mix.right.z"], out[p + "mix.right.z.b"] = (R, W), (R,)
                out[p + "mix.right.x"], out[p + "mix.right.x.b"] = (R, W), (R,)
                out[p + "mix.right.g"], out[p + "mix.right.o"] = (R, W), (W, R)
            if l.mlp:
                out[p + "mlp.up"], out[p + "mlp.down"] = (l.ff, W), (W, l.ff)
        out["final.norm"] = (W,)
        return out


def synthetic_weights(spec: VokepelSpec, seed: int = 0, device="cpu") -> dict:
    """Seeded random-init checkpoint (bf16 tensors on `device`): matrices ~ 1 / sqrt(in), gains around 1, small positive distance
    penalties, a head-mixing matrix near the identity, sinks and biases of order 1; activations stay O(1) through the stack."""
    g = torch.Generator(device=device).manual_seed(seed)

    def randn(shape):
        return torch.randn(shape, generator=g, device=device)
    ck = {}
    for name, shape in spec.tensor_shapes().items():
        if name.endswith("norm1") or name.endswith("norm2") or name.endswith(".norm"):
            t = 1.0 + 0.1 * randn(shape)
        elif name.endswith("mix.r1"):
            t = 0.3 * torch.rand(shape, generator=g, device=device)
        elif name.endswith("mix.r2"):
            t = 0.2 + 0.8 * torch.rand(shape, generator=g, device=device)
        elif name.endswith("mix.talk"):
            t = torch.eye(shape[0], device=device) + 0.2 * randn(shape)
        elif name.endswith(".sink") or name.endswith(".b"):
            t = 0.5 * randn(shape)
        elif name == "loop.step":
            t = 0.1 * randn(shape)
        elif name == "embed":
            t = randn(shape)
        else:
            t = randn(shape) / math.sqrt(shape[-1])
        ck[name] = t.to(torch.bfloat16)
    return ck


class VokepelForCausalLM:
    """The executor handle: weights, paged key/value caches and recurrent-state slots of every layer run, and workspaces live in
    the library."""

    architecture = "Vokepel"

    def __init__(self, spec: VokepelSpec, dtype: str = "bfloat16", block_size: int = 16, num_blocks: int = 256, max_tokens: int = 2048,
                 max_seqs: int = 64, device: int = 0):
        if dtype not in ("bfloat16", "float32"):
            raise ValueError(f"Vokepel runs in bfloat16 or float32, not `{dtype}`")
        self.spec, self.dtype = spec, dtype
        self.block_size, self.num_blocks, self.max_tokens, self.max_seqs = block_size, num_blocks, max_tokens, max_seqs
        self.vocab_size = spec.vocab
        self.state_slots = max_seqs          # the engine hands one to every live sequence
        self.device = torch.device("cuda", device)
        a, b, times = spec.loop or (0, 0, 0)
        cfg = VokepelConfig(spec.vocab, spec.width, len(spec.layers), spec.norm_eps, spec.residual_mult, spec.logit_scale, spec.logit_softcap,
                            a, b, times, VMX_F32 if dtype == "float32" else VMX_BF16, block_size, num_blocks, max_tokens, max_seqs, self.state_slots)
        layers = (VokepelLayerConfig * len(spec.layers))()
        for i, l in enumerate(spec.layers):
            layers[i] = VokepelLayerConfig(MIXERS[l.mixer], l.heads, l.kv_heads, l.dim, l.vdim, l.window, l.scale, l.softcap, l.rot_dims, l.rot_base,
                                           l.gru_width, l.left_scale, l.right_scale, MLPS[l.mlp], l.ff)
        self._h = C.c_void_p()
        check(lib.vmx_vokepel_create(C.byref(cfg), layers, C.byref(self._h)))
        self.num_layer_runs = lib.vmx_vokepel_num_layer_runs(self._h)

    @classmethod
    def from_pretrained(cls, model_dir, dtype: str = "bfloat16", **kw) -> "VokepelForCausalLM":
        cfg = json.loads((Path(model_dir) / "config.json").read_text())
        model = cls(VokepelSpec.from_config(cfg), dtype=dtype, **kw)
        model.load_checkpoint(model_dir)
        return model

    def close(self):
        if self._h:
            lib.vmx_vokepel_destroy(self._h)
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
            check(lib.vmx_vokepel_load_tensor(self._h, name.encode(), t.ctypes.data, t.nbytes, self._stream()))
            return
        assert t.dtype == torch.bfloat16, f"{name}: bf16 expected, got {t.dtype}"
        t = t.contiguous()
        check(lib.vmx_vokepel_load_tensor(self._h, name.encode(), t.data_ptr(), t.numel() * 2, self._stream()))

    def load_state(self, tensors: dict) -> None:
        for name, t in tensors.items():
            self.load_tensor(name, t)
        self.check_loaded()

    def check_loaded(self) -> None:
        if lib.vmx_vokepel_missing_tensors(self._h) != 0:
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
                    raise ValueError(f"{model_dir}: tensor `{name}` is {dtype}; Vokepel checkpoints hold bf16")
                m = re.fullmatch(r"l(\d+)\.norm2", name)
                if m and int(m.group(1)) < len(self.spec.layers) and self.spec.layers[int(m.group(1))].mlp is None:
                    continue                 # the norm of a feed-forward this layer does not have
                if name in ("loop.in", "loop.step") and not self.spec.loop:
                    continue                 # the entry of a loop the configuration does not have
                self.load_tensor(name, ck.get(name))
        finally:
            ck.close()
        self.check_loaded()

    def forward(self, tokens, prev_tokens, positions, slots, seq_ids, block_tables, logit_rows=None, want_logits: bool = True,
                want_greedy: bool = False, layer_trace: bool = False, seq_starts=None, state_slots=None):
        """One packed step; every argument an int32 CUDA tensor ([T] each, block_tables [S, max_blocks], seq_starts [S + 1],
        state_slots [S], logit_rows [n]); prev_tokens is not used by this design.
        Returns (logits f32 [n, vocab] or None, greedy ids int32 [n] or None, trace f32 [layer runs, T, width] or None)."""
        if seq_starts is None or state_slots is None:
            raise ValueError("Vokepel carries recurrent state: the step needs seq_starts and state_slots")
        T = tokens.numel()
        S = seq_starts.numel() - 1           # the sequences of THIS step; the block table may hold more rows
        if S < 1 or state_slots.numel() != S or block_tables.shape[0] < S:
            raise ValueError(f"Vokepel: {S} sequences by seq_starts, {state_slots.numel()} state slots, {block_tables.shape[0]} block-table rows")
        if not all(a.numel() == T for a in (positions, slots, seq_ids)):
            raise ValueError("Vokepel: tokens, positions, slots and seq_ids must have one entry per token")
        n = 0 if logit_rows is None else logit_rows.numel()
        logits = torch.empty((n, self.spec.vocab), dtype=torch.float32, device=self.device) if n else None
        ids = torch.empty(n, dtype=torch.int32, device=self.device) if (n and want_greedy) else None
        trace = torch.empty((self.num_layer_runs, T, self.spec.width), dtype=torch.float32, device=self.device) if layer_trace else None
        check(lib.vmx_vokepel_forward(self._h, tokens.data_ptr(), positions.data_ptr(), slots.data_ptr(), seq_ids.data_ptr(), T,
                                      block_tables.data_ptr(), S, block_tables.shape[1], seq_starts.data_ptr(),
                                      state_slots.data_ptr(), None if not n else logit_rows.data_ptr(), n,
                                      None if logits is None else logits.data_ptr(), None if ids is None else ids.data_ptr(),
                                      None if trace is None else trace.data_ptr(), self._stream()))
        return (logits if want_logits else None), ids, trace

"""Model registry: which executor driver serves a checkpoint directory, chosen by its config.json.

`architecture` (or the first entry of Hugging Face's `architectures`) names the model class; `load_model` builds the driver,
sizes its paged cache and loads the weights, and returns it wrapped for `vllm_rust_amd.engine.Engine`.
"""
from __future__ import annotations

import json
from pathlib import Path

REGISTRY = {}


def register(name: str):
    def deco(fn):
        REGISTRY[name] = fn
        return fn
    return deco


def architecture_of(model_dir) -> str:
    cfg = json.loads((Path(model_dir) / "config.json").read_text())
    arch = cfg.get("architecture") or (cfg.get("architectures") or [None])[0]
    if arch is None:
        raise ValueError(f"{model_dir}/config.json names no architecture")
    return arch


def _cache_geometry(max_tokens: int, max_seqs: int, block_size: int):
    # every live sequence may leave its last block partly used
    return (max_tokens + block_size - 1) // block_size + max_seqs + 1


@register("Gesutar")
def _load_gesutar(model_dir, dtype, max_tokens, max_seqs, block_size, device):
    from .gesutar import GesutarForCausalLM
    return GesutarForCausalLM.from_pretrained(model_dir, dtype=dtype, block_size=block_size,
                                              num_blocks=_cache_geometry(max_tokens, max_seqs, block_size), max_tokens=max_tokens,
                                              max_seqs=max_seqs, device=device)


@register("Gupuvik")
def _load_gupuvik(model_dir, dtype, max_tokens, max_seqs, block_size, device):
    from .gupuvik import GupuvikForCausalLM
    return GupuvikForCausalLM.from_pretrained(model_dir, dtype=dtype, block_size=block_size,
                                              num_blocks=_cache_geometry(max_tokens, max_seqs, block_size), max_tokens=max_tokens,
                                              max_seqs=max_seqs, device=device)


@register("Vokepel")
def _load_vokepel(model_dir, dtype, max_tokens, max_seqs, block_size, device):
    from .vokepel import VokepelForCausalLM
    return VokepelForCausalLM.from_pretrained(model_dir, dtype=dtype, block_size=block_size,
                                              num_blocks=_cache_geometry(max_tokens, max_seqs, block_size), max_tokens=max_tokens,
                                              max_seqs=max_seqs, device=device)


@register("Gezozen")
def _load_gezozen(model_dir, dtype, max_tokens, max_seqs, block_size, device):
    from .gezozen import GezozenForCausalLM
    return GezozenForCausalLM.from_pretrained(model_dir, dtype=dtype, block_size=block_size,
                                              num_blocks=_cache_geometry(max_tokens, max_seqs, block_size), max_tokens=max_tokens,
                                              max_seqs=max_seqs, device=device)


@register("Qwen3ForCausalLM")
def _load_qwen3(model_dir, dtype, max_tokens, max_seqs, block_size, device):
    """AWQ / GPTQ / EXL3 Qwen3 checkpoints (the quantization is detected from the directory)."""
    from . import checkpoint as ck
    from .engine import PackedQwen3
    from .qwen3 import QuantizedQwen3ForCausalLM, Qwen3Spec
    if dtype != "bfloat16":
        raise NotImplementedError("the Qwen3 executor runs in bfloat16 (fp16 for EXL3 checkpoints)")
    cfg = json.loads((Path(model_dir) / "config.json").read_text())
    det = ck.detect_from_directory(model_dir)
    spec = Qwen3Spec(cfg["hidden_size"], cfg["num_hidden_layers"], cfg["num_attention_heads"], cfg["num_key_value_heads"],
                     cfg.get("head_dim", cfg["hidden_size"] // cfg["num_attention_heads"]), cfg["intermediate_size"], cfg["vocab_size"],
                     rms_norm_eps=cfg.get("rms_norm_eps", 1e-6), rope_theta=cfg.get("rope_theta", 1e6),
                     max_position=min(cfg.get("max_position_embeddings", 4096), max(max_tokens, 4096)), group_size=det.group_size or 128,
                     tie_word_embeddings=bool(cfg.get("tie_word_embeddings", False)), block_size=block_size,
                     num_blocks=_cache_geometry(max_tokens, max_seqs, block_size), max_batch=min(max_seqs, 16), max_seq_len=max_tokens,
                     max_prefill_tokens=max_tokens, act_dtype="f16" if det.method == "exl3" else "bf16")
    model = QuantizedQwen3ForCausalLM(spec, device)
    loader = {"awq": ck.load_qwen3_awq_checkpoint, "awq_marlin": ck.load_qwen3_awq_checkpoint, "gptq": ck.load_qwen3_gptq_checkpoint,
              "gptq_marlin": ck.load_qwen3_gptq_checkpoint, "exl3": ck.load_qwen3_exl3_checkpoint}.get(det.method)
    if loader is None:
        raise NotImplementedError(f"{model_dir}: no loader for quantization `{det.method}`")
    loader(model, model_dir)
    return PackedQwen3(model)


def load_model(model_dir, dtype: str = "bfloat16", max_tokens: int = 2048, max_seqs: int = 16, block_size: int = 16, device: int = 0):
    arch = architecture_of(model_dir)
    if arch not in REGISTRY:
        raise NotImplementedError(f"architecture `{arch}` is not registered (known: {', '.join(sorted(REGISTRY))})")
    return REGISTRY[arch](model_dir, dtype, max_tokens, max_seqs, block_size, device)

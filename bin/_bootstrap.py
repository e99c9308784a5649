"""Shared start-up of the command-line tools: compile the HIP library on first use (a fresh checkout holds sources only)."""
import json
import os
import subprocess
import sys
from pathlib import Path

ROOT = Path(__file__).resolve().parent.parent
LIB = ROOT / "vllm-rust_amd" / "lib"
# architectures (config.json) whose kernels build as a library of their own (csrc/Makefile FAMILY=...)
FAMILY_OF = {"Vokepel": "vokepel", "Gezozen": "gezozen"}


def _family(model_dir):
    try:
        cfg = json.loads((Path(model_dir) / "config.json").read_text())
    except (OSError, ValueError):
        return None
    return FAMILY_OF.get(cfg.get("architecture") or (cfg.get("architectures") or [None])[0])


def ensure_built(model_dir=None) -> None:
    """The whole library if it is there; else the one-family library of the model's architecture where the Makefile has one
    (built now if missing: only the sources that family runs), else the whole library (built now)."""
    if (LIB / "libvmx.so").exists() and not os.environ.get("VMX_LIB_VARIANT"):
        return
    jobs = os.environ.get("MAX_JOBS") or str(min(16, os.cpu_count() or 4))
    family = _family(model_dir) if model_dir else None
    if os.environ.get("VMX_LIB_VARIANT"):
        return                       # the caller chose a build
    if family:
        if not (LIB / f"libvmx_{family}.so").exists():
            print(f"building libvmx_{family}.so ...", file=sys.stderr, flush=True)
            subprocess.run(["make", "-C", str(ROOT / "vllm-rust_amd" / "csrc"), "-j" + jobs, f"FAMILY={family}"], check=True, stdout=sys.stderr)
        os.environ["VMX_LIB_VARIANT"] = family
        return
    print("building libvmx.so ...", file=sys.stderr, flush=True)
    subprocess.run(["make", "-C", str(ROOT / "vllm-rust_amd" / "csrc"), "-j" + jobs], check=True, stdout=sys.stderr)


def import_package(model_dir=None):
    """Build if needed, then import the package from this checkout."""
    ensure_built(model_dir)
    if str(ROOT) not in sys.path:
        sys.path.insert(0, str(ROOT))
    import vllm_rust_amd
    return vllm_rust_amd

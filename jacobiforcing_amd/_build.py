"""Compiles the package's HIP libraries for gfx950 with hipcc (cross-compiles without a GPU).  ``libjacobiforcing.so`` is the
Jacobi loop body; ``libjf_layers.so`` and ``libjf_layers_seq.so`` hold the layer kernels of the models whose forward is not stock
PyTorch.  Each is built from its own sources only, so a process that needs one does not wait for the others."""
from __future__ import annotations

import os
import shutil
import subprocess
import tempfile
from pathlib import Path

_PKG = Path(__file__).resolve().parent
ROOT = _PKG.parent
CSRC = _PKG / "csrc"
LIB_DIR = _PKG / "lib"
# every translation unit is compiled without packed-fp32 instructions (the flag is for the device pass; the host pass warns)
HIP_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument"]

# The layer kernels come in two libraries, so that a model compiles (at the first call of a fresh checkout) only what it launches:
# "layers" = norms, convolution, attention and its input / output stages; "layers_seq" = the recurrent mixers and the routed experts.
LAYER_GROUPS = {
    "layers": ["jl_error", "jl_norm", "jl_conv", "jl_headnorm", "jl_latent", "jl_attn_sweep", "jl_attn"],
    "layers_seq": ["jl_error", "jl_retention", "jl_delta", "jl_moe"],
}
LAYERS_HEADERS = [CSRC / "layers" / "jl_common.h", ROOT / "include" / "jf_layers.h"]


def layer_lib(group: str) -> Path:
    return LIB_DIR / f"libjf_{group}.so"


def layer_sources(group: str):
    return [CSRC / "layers" / f"{stem}.hip" for stem in LAYER_GROUPS[group]]


def hipcc() -> str:
    return shutil.which("hipcc") or "/opt/rocm/bin/hipcc"


def stale(target: Path, deps) -> bool:
    return (not target.exists()) or target.stat().st_mtime < max(Path(d).stat().st_mtime for d in deps)


def build_layers(force: bool = False, groups=None):
    """Every group of ``groups`` (default: all): one object per source, compiled side by side, linked into ``lib/libjf_<group>.so``
    (written under a temporary name and renamed, so that a process that starts meanwhile never loads half a file)."""
    LIB_DIR.mkdir(parents=True, exist_ok=True)
    todo = [g for g in (groups or LAYER_GROUPS) if force or stale(layer_lib(g), layer_sources(g) + LAYERS_HEADERS)]
    if not todo:
        return [layer_lib(g) for g in (groups or LAYER_GROUPS)]
    with tempfile.TemporaryDirectory(dir=LIB_DIR) as tmp:
        inc = [f"-I{ROOT / 'include'}", f"-I{CSRC / 'layers'}"]
        stems = sorted({s for g in todo for s in LAYER_GROUPS[g]}, key=lambda s: s != "jl_attn")      # the longest compile starts first
        jobs = [(subprocess.Popen([hipcc(), *HIP_FLAGS, *inc, "-c", str(CSRC / "layers" / f"{s}.hip"), "-o", f"{tmp}/{s}.o"], stderr=subprocess.PIPE,
                                  text=True), s) for s in stems]
        for p, s in jobs:
            _, err = p.communicate()
            if p.returncode:
                raise RuntimeError(f"hipcc failed on {s}.hip:\n{err[-4000:]}")
        for g in todo:
            out = f"{tmp}/libjf_{g}.so"
            subprocess.check_call([hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", *[f"{tmp}/{s}.o" for s in LAYER_GROUPS[g]], "-o", out])
            os.replace(out, layer_lib(g))
    return [layer_lib(g) for g in (groups or LAYER_GROUPS)]

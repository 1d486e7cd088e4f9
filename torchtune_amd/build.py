"""Compile the HIP sources in ``torchtune_amd/csrc`` into ``torchtune_amd/lib/libtorchtune_amd.so`` for gfx950.

The library is a plain C-ABI shared object (see ``include/torchtune_amd.h``); it links against the HIP
runtime only, never against torch.  ``python -m torchtune_amd.build`` rebuilds it.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG = Path(__file__).resolve().parent
CSRC = PKG / "csrc"
LIB_DIR = PKG / "lib"
LIB_PATH = LIB_DIR / "libtorchtune_amd.so"
SOURCES = ["capi.hip", "nf4_codec.hip", "fake_quant.hip", "nf4_gemm.hip", "nf4_gemm_rs.hip", "nf4_gemm_dense.hip", "gemm_tn.hip", "nf4_small_m.hip", "lora_skinny.hip", "lora_group.hip", "qlora_linear.hip", "nf4_merge.hip", "neighbours.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fno-fast-math",
    "-ffp-contract=off",  # quantisation results must not depend on fma contraction
    "-fhip-fp32-correctly-rounded-divide-sqrt",
    "-fno-gpu-flush-denormals-to-zero",
    # packed fp32 VALU ops are kept out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall",
    "-Wno-unused-function",
]


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found: the HIP toolchain (ROCm) is required to build torchtune_amd")
    return exe


def _compile(src: str, obj_dir: Path) -> Path:
    obj = obj_dir / (Path(src).stem + ".o")
    cmd = [hipcc(), *HIPCC_FLAGS, "-c", str(CSRC / src), "-o", str(obj)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{proc.stdout}\n{proc.stderr}")
    return obj


def build(verbose: bool = False) -> Path:
    """Compile every source and link the shared library. Always recompiles."""
    obj_dir = PKG / "build"
    obj_dir.mkdir(exist_ok=True)
    LIB_DIR.mkdir(exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(len(SOURCES), 8)) as pool:
        objs = list(pool.map(lambda s: _compile(s, obj_dir), SOURCES))
    tmp = LIB_PATH.with_suffix(".so.tmp")
    cmd = [hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(tmp), *map(str, objs)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stdout}\n{proc.stderr}")
    os.replace(tmp, LIB_PATH)
    if verbose:
        print(f"built {LIB_PATH}")
    return LIB_PATH


if __name__ == "__main__":
    build(verbose=True)
    sys.exit(0)

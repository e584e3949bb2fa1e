"""Build recipe for ``libnf_cdna4.so`` (the C-ABI library of hand-written gfx950 kernels).

``python -m triton_helpers_amd.build`` cross-compiles every ``csrc/*.hip`` with
``hipcc --offload-arch=gfx950`` (no GPU needed) and links them into
``triton_helpers_amd/libnf_cdna4.so`` next to this file.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path
from typing import List

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
INCLUDE = PKG_DIR.parent / "include"
LIB_PATH = PKG_DIR / "libnf_cdna4.so"
BUILD_DIR = PKG_DIR / "build"

ARCH = "gfx950"
COMMON_FLAGS = [
    f"--offload-arch={ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-munsafe-fp-atomics",
    # keep the compiler from emitting packed-fp32 VALU forms
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    f"-I{INCLUDE}",
    f"-I{CSRC}",
]
# Files whose float arithmetic must not be contracted into FMAs (bit-exact cell / weight math).
NO_CONTRACT = {"hash_encoding.hip", "hash_encoding_bwd_scan.hip", "hash_encoding_bwd_bin.hip", "hash_encoding_bwd_static.hip", "hash_check_host.hip"}
# Files whose MFMA results feed vector ALU work directly: keep them in architectural VGPRs instead of
# bouncing every result through an accumulation register.
MFMA_VGPR_FORM = {"fused_mlp.hip", "fused_mlp_bwd2.hip", "fused_mlp_bwdn.hip", "fused_mlp_bwd2_w8.hip", "fused_mlp_bwd2_ws.hip", "fused_mlp_fwd2.hip", "reversible_mlp.hip"}


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; a ROCm toolchain is required to build libnf_cdna4.so")
    return exe


def _run(cmd: List[str], verbose: bool) -> None:
    if verbose:
        print("+", " ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"command failed ({proc.returncode}): {' '.join(cmd)}\n{out}")
    if verbose and out.strip():
        print(out, flush=True)


def sources() -> List[Path]:
    return sorted(CSRC.glob("*.hip"))


def build(verbose: bool = True, jobs: int = 8) -> Path:
    """Compile all kernels and link the shared library; returns its path."""
    hipcc = _hipcc()
    BUILD_DIR.mkdir(exist_ok=True)
    objs = []
    cmds = []
    for src in sources():
        obj = BUILD_DIR / (src.stem + ".o")
        flags = list(COMMON_FLAGS)
        if src.name in NO_CONTRACT:
            flags.append("-ffp-contract=off")
        if src.name in MFMA_VGPR_FORM:
            flags += ["-mllvm", "-amdgpu-mfma-vgpr-form"]
        cmds.append([hipcc, *flags, "-c", str(src), "-o", str(obj)])
        objs.append(obj)
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        list(ex.map(lambda c: _run(c, verbose), cmds))
    tmp = LIB_PATH.with_suffix(".so.tmp")
    _run([hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", *map(str, objs), "-o", str(tmp)], verbose)
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    path = build(verbose="-q" not in sys.argv)
    print(f"built {path}")

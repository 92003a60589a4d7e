"""Build recipe for the HIP library: hipcc on csrc/*.hip -> csrc/libspeed3r_hip.so (gfx950 only).

Run as ``python -m speed3r_amd.build``.  The library is built in-tree so that it travels with
the source tree; nothing is installed.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from pathlib import Path

CSRC = Path(__file__).resolve().parent / "csrc"
LIB_NAME = "libspeed3r_hip.so"
SOURCES = ["api.hip", "pool_merge.hip", "topk.hip", "attn_simple.hip", "select_pipe.hip", "compressed_mfma.hip", "norm_rope.hip", "qkv_prepass.hip", "layer_norm.hip", "attn_bwd.hip", "select_b16.hip", "key_lists.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    # keep the compiler from forming packed-fp32 VALU instructions out of scalar float code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-value",
]


def hipcc_path() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (set HIPCC or install ROCm under /opt/rocm)")


def library_path() -> Path:
    return CSRC / LIB_NAME


def build_library(verbose: bool = True, extra_flags=()) -> Path:
    """Compile every kernel source into one shared library; raises on failure."""
    out = library_path()
    cmd = [hipcc_path(), *HIPCC_FLAGS, *extra_flags, *[str(CSRC / s) for s in SOURCES], "-o", str(out)]
    if verbose:
        print("[speed3r_amd.build]", " ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass warns that it does not know the packed-fp32 feature; that is expected
    err = "\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + err)
    if verbose and err.strip():
        print(err, file=sys.stderr)
    return out


if __name__ == "__main__":
    print(build_library())

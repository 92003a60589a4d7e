"""Build recipe for the HIP library: hipcc on csrc/*.hip -> csrc/libspeed3r_hip.so (gfx950 only).

Run as ``python -m speed3r_amd.build`` (``--changed``: recompile only sources newer than their objects).  The
library is built in-tree so that it travels with the source tree; nothing is installed.
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


def _filter_stderr(text: str) -> str:
    # the host pass warns that it does not know the packed-fp32 feature; that is expected
    return "\n".join(l for l in text.splitlines() if "packed-fp32-ops" not in l)


def build_library(verbose: bool = True, extra_flags=(), sources=None, out=None, jobs: int = 0, only_changed: bool = False) -> Path:
    """Compile every kernel source (one hipcc process per file, ``jobs`` at a time) and link the objects into one
    shared library; raises on failure.  ``only_changed`` keeps objects newer than their source and every header
    (a developer's shortcut; the default compiles everything)."""
    from concurrent.futures import ThreadPoolExecutor

    out = Path(out) if out is not None else library_path()
    sources = [Path(s) if os.path.isabs(str(s)) else CSRC / s for s in (sources or SOURCES)]
    objdir = CSRC / "build"
    objdir.mkdir(exist_ok=True)
    compile_flags = [f for f in HIPCC_FLAGS if f != "-shared"]
    headers_mtime = max(h.stat().st_mtime for h in CSRC.glob("*.h"))
    tag = "" if not extra_flags else "_" + "".join(c if c.isalnum() else "_" for c in "".join(extra_flags))
    jobs = jobs or min(len(sources), max(1, (os.cpu_count() or 2)), 16)

    def compile_one(src: Path):
        obj = objdir / (src.stem + tag + ".o")
        if only_changed and obj.exists() and obj.stat().st_mtime > max(src.stat().st_mtime, headers_mtime):
            return obj, 0, ""
        cmd = [hipcc_path(), *compile_flags, *extra_flags, "-I", str(CSRC), "-c", str(src), "-o", str(obj)]
        if verbose:
            print("[speed3r_amd.build]", " ".join(cmd), flush=True)
        res = subprocess.run(cmd, capture_output=True, text=True)
        return obj, res.returncode, _filter_stderr(res.stderr)

    with ThreadPoolExecutor(max_workers=jobs) as pool:
        results = list(pool.map(compile_one, sources))
    failed = [(o, e) for o, rc, e in results if rc != 0]
    if failed:
        raise RuntimeError("hipcc failed:\n" + "\n".join(e for _, e in failed))
    for _, _, e in results:
        if verbose and e.strip():
            print(e, file=sys.stderr)
    cmd = [hipcc_path(), "--offload-arch=gfx950", "-shared", "-fPIC", *[str(o) for o, _, _ in results], "-o", str(out)]
    if verbose:
        print("[speed3r_amd.build]", " ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("hipcc (link) failed:\n" + _filter_stderr(res.stderr))
    return out


if __name__ == "__main__":
    print(build_library(only_changed="--changed" in sys.argv[1:]))

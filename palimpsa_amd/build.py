"""Build libpalimpsa_hip.so (gfx950) from palimpsa_amd/csrc with hipcc.

Usage: ``python -m palimpsa_amd.build [--force]``.  The library is written
in-tree (palimpsa_amd/lib/) and carries no torch dependency: it is plain HIP
behind the C ABI of include/palimpsa_hip.h.
"""
from __future__ import annotations

import concurrent.futures
import os
import shutil
import subprocess
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
LIB_DIR = os.path.join(PKG_DIR, "lib")
OBJ_DIR = os.path.join(LIB_DIR, "obj")
LIB_PATH = os.path.join(LIB_DIR, "libpalimpsa_hip.so")

ARCH = "gfx950"
# packed-fp32 VALU forms are switched off on purpose: hipcc -O3 would otherwise
# turn ordinary float code into v_pk_*_f32.
CXXFLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # MFMA results are consumed by VALU epilogues: keep them in arch VGPRs instead of
    # AccVGPRs that would need a v_accvgpr_read per element
    "-mllvm", "-amdgpu-mfma-vgpr-form",
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; a ROCm toolchain is required to build palimpsa_amd")
    return exe


def sources():
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def _headers():
    hs = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")]
    hs.append(os.path.join(os.path.dirname(PKG_DIR), "include", "palimpsa_hip.h"))
    return hs


def _compile_one(src: str, force: bool) -> str:
    obj = os.path.join(OBJ_DIR, os.path.basename(src)[:-4] + ".o")
    newest_dep = max(os.path.getmtime(p) for p in [src] + _headers())
    if not force and os.path.exists(obj) and os.path.getmtime(obj) >= newest_dep:
        return obj
    cmd = [_hipcc()] + CXXFLAGS + ["-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{r.stdout}\n{r.stderr}")
    noise = ("packed-fp32-ops", "-target-feature")
    warn = [ln for ln in r.stderr.splitlines() if "warning" in ln and not any(n in ln for n in noise)]
    if warn:
        sys.stderr.write("\n".join(warn) + "\n")
    return obj


def build(force: bool = False, jobs: int = 8) -> str:
    """Compile every .hip under csrc/ and link the shared library.  Returns its path."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    srcs = sources()
    with concurrent.futures.ThreadPoolExecutor(max_workers=max(1, min(jobs, len(srcs)))) as ex:
        objs = list(ex.map(lambda s: _compile_one(s, force), srcs))
    if (not force and os.path.exists(LIB_PATH)
            and os.path.getmtime(LIB_PATH) >= max(os.path.getmtime(o) for o in objs)):
        return LIB_PATH
    cmd = [_hipcc(), f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", LIB_PATH] + objs
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stdout}\n{r.stderr}")
    return LIB_PATH


if __name__ == "__main__":
    p = build(force="--force" in sys.argv)
    print(p)

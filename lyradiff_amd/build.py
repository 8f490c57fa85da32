"""Builds liblyraquant.so (hand-written HIP for gfx950 behind the C ABI of include/lyraquant.h) and libth_lyradiff.so
(the torch custom classes over it).

    python -m lyradiff_amd.build [--force]

Every .hip/.cpp under csrc/ is compiled with hipcc for gfx950 only (cross-compiles without a
GPU) and linked in-tree into lyradiff_amd/liblyraquant.so.
"""
from __future__ import annotations

import concurrent.futures as cf
import os
import subprocess
import sys

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
OBJ = os.path.join(PKG, "csrc", "build")
LIB = os.path.join(PKG, "liblyraquant.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17",
    "-ffp-contract=off",  # the quantisation formulas are specified without fused multiply-add
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option",
    "-I", os.path.join(ROOT, "include"), "-I", CSRC,
]


def sources():
    return sorted(f for f in os.listdir(CSRC) if f.endswith((".hip", ".cpp")))


def _deps_mtime(path: str, seen=None) -> float:
    """Newest modification time among `path` and the project headers it includes, directly or not."""
    seen = set() if seen is None else seen
    if path in seen or not os.path.exists(path):
        return 0.0
    seen.add(path)
    newest = os.path.getmtime(path)
    with open(path, errors="replace") as f:
        for line in f:
            line = line.strip()
            if line.startswith("#include \""):
                name = line.split('"')[1]
                for d in (os.path.dirname(path), CSRC, os.path.join(ROOT, "include")):
                    newest = max(newest, _deps_mtime(os.path.join(d, name), seen))
    return newest


def _compile(src: str, force: bool) -> str:
    obj = os.path.join(OBJ, src + ".o")
    path = os.path.join(CSRC, src)
    if not force and os.path.exists(obj) and os.path.getmtime(obj) >= _deps_mtime(path):
        return obj
    cmd = [HIPCC, *FLAGS, "-c", path, "-o", obj]
    if src.endswith(".cpp"):
        cmd = [HIPCC, "-x", "c++", "-O2", "-fPIC", "-std=c++17", "-I", os.path.join(ROOT, "include"), "-c", path, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{r.stdout}\n{r.stderr}")
    return obj


def build(force: bool = False, jobs: int | None = None) -> str:
    os.makedirs(OBJ, exist_ok=True)
    jobs = jobs or min(8, os.cpu_count() or 1)
    with cf.ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(lambda s: _compile(s, force), sources()))
    if force or not os.path.exists(LIB) or any(os.path.getmtime(o) > os.path.getmtime(LIB) for o in objs):
        cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"link failed:\n{r.stdout}\n{r.stderr}")
    build_compat_check(force)
    build_torch_classes(force)
    return LIB


TH_LIB = os.path.join(PKG, "libth_lyradiff.so")


def build_torch_classes(force: bool = False) -> str:
    """Compiles th_op/th_lyradiff.cpp (torch.classes.lyradiff.*, host code only) against PyTorch's headers and links it to
    liblyraquant.so next to it."""
    import torch

    src = os.path.join(PKG, "th_op", "th_lyradiff.cpp")
    newest = max(os.path.getmtime(f) for f in (src, LIB, os.path.join(ROOT, "include", "lyraquant.h")))
    if not force and os.path.exists(TH_LIB) and os.path.getmtime(TH_LIB) >= newest:
        return TH_LIB
    tdir = os.path.dirname(torch.__file__)
    cmd = [os.environ.get("CXX", "g++"), "-std=c++17", "-O2", "-fPIC", "-shared", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}", "-Wno-deprecated-declarations",
           "-I", os.path.join(ROOT, "include"), "-I", os.path.join(tdir, "include"),
           "-I", os.path.join(tdir, "include", "torch", "csrc", "api", "include"), "-I", "/opt/rocm/include",
           src, "-o", TH_LIB, "-L", os.path.join(tdir, "lib"), "-ltorch", "-ltorch_cpu", "-lc10", "-lc10_hip", "-ltorch_hip",
           "-L", PKG, "-llyraquant", "-Wl,-rpath,$ORIGIN"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"libth_lyradiff.so build failed:\n{r.stdout}\n{r.stderr}")
    return TH_LIB


def build_compat_check(force: bool = False) -> list:
    """Compiles the reference-style C++ call-site programs under tests/cpp against the library."""
    exes = []
    hdrs = [os.path.join(ROOT, "include", h) for h in ("lyradiff_compat.h", "lyradiff_layers.h", "lyraquant.h")]
    for name in ("compat_check", "layers_check", "flux_fp8_check"):
        src = os.path.join(ROOT, "tests", "cpp", name + ".cpp")
        exe = os.path.join(ROOT, "tests", "cpp", name)
        if not os.path.exists(src):
            continue
        newest = max(os.path.getmtime(f) for f in [src, LIB, *hdrs])
        if force or not os.path.exists(exe) or os.path.getmtime(exe) < newest:
            cmd = [HIPCC, "--offload-arch=gfx950", "-O2", "-std=c++17", "-ffp-contract=off", "-Wno-unused-command-line-argument",
                   "-I", os.path.join(ROOT, "include"), src, "-o", exe, "-L", PKG, "-llyraquant",
                   "-Wl,-rpath,$ORIGIN/../../lyradiff_amd"]
            r = subprocess.run(cmd, capture_output=True, text=True)
            if r.returncode != 0:
                raise RuntimeError(f"{name} build failed:\n{r.stdout}\n{r.stderr}")
        exes.append(exe)
    return exes


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))

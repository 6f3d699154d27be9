"""Builds ``siirl_amd/lib/libsiirl_hip.so`` from ``siirl_amd/csrc/*.hip`` with hipcc for gfx950, and
``siirl_amd/lib/libsiirl_torch.so`` (the ``TORCH_LIBRARY(siirl_hip, ...)`` layer, host-only C++ over the C ABI of the
first) from ``siirl_amd/csrc/torch_ops.cpp`` with g++ against the installed torch's headers.

Usage: ``python -m siirl_amd.build [--force]``.  The libraries are built in-tree so that they travel with
the source tree to a GPU machine; nothing is compiled at import time."""

from __future__ import annotations

import argparse
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG = Path(__file__).resolve().parent
CSRC = PKG / "csrc"
LIBDIR = PKG / "lib"
LIBNAME = "libsiirl_hip.so"
TORCH_LIBNAME = "libsiirl_torch.so"
CXX = os.environ.get("CXX", "g++")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
ARCH = "gfx950"
# -packed-fp32-ops: keep the compiler from forming v_pk_{add,mul,fma}_f32 out of scalar float code.
CXXFLAGS = ["-O3", "-std=c++17", "-fPIC", f"--offload-arch={ARCH}", "-Xclang", "-target-feature", "-Xclang",
            "-packed-fp32-ops", "-Wno-unused-command-line-argument", "-fno-gpu-rdc"]
# per-file additions: the numpy-emulating group statistics and the GAE recurrences must not be contracted into FMAs
EXTRA = {"group_ops.hip": ["-ffp-contract=off"], "gae.hip": ["-ffp-contract=off"],
         "reward.hip": ["-ffp-contract=off"], "marft_gae.hip": ["-ffp-contract=off"]}


def sources():
    return sorted(CSRC.glob("*.hip"))


def _stale(out: Path, deps) -> bool:
    if not out.exists():
        return True
    t = out.stat().st_mtime
    return any(Path(d).stat().st_mtime > t for d in deps)


def _filter(stderr: str) -> str:
    keep = [ln for ln in stderr.splitlines() if "packed-fp32-ops" not in ln and "is not a recognized feature" not in ln]
    return "\n".join(keep)


def build(force: bool = False, verbose: bool = True) -> Path:
    LIBDIR.mkdir(exist_ok=True)
    objdir = PKG / "build"
    objdir.mkdir(exist_ok=True)
    headers = list(CSRC.glob("*.hpp")) + list((PKG.parent / "include").glob("*.h"))
    jobs = []
    for src in sources():
        obj = objdir / (src.stem + ".o")
        if force or _stale(obj, [src, *headers]):
            jobs.append((src, obj))

    def compile_one(job):
        src, obj = job
        cmd = [HIPCC, *CXXFLAGS, *EXTRA.get(src.name, []), "-c", str(src), "-o", str(obj)]
        r = subprocess.run(cmd, capture_output=True, text=True)
        return src, r.returncode, _filter(r.stderr)

    with ThreadPoolExecutor(max_workers=min(8, max(1, len(jobs)))) as ex:
        for src, rc, err in ex.map(compile_one, jobs):
            if verbose:
                print(f"[siirl_amd.build] hipcc {src.name}: {'ok' if rc == 0 else 'FAILED'}", flush=True)
            if err.strip() and (rc != 0 or verbose):
                print(err, file=sys.stderr)
            if rc != 0:
                raise RuntimeError(f"hipcc failed on {src}")
    out = LIBDIR / LIBNAME
    objs = [str(objdir / (s.stem + ".o")) for s in sources()]
    if force or jobs or not out.exists():
        cmd = [HIPCC, "-shared", "-fPIC", f"--offload-arch={ARCH}", "-fno-gpu-rdc", "-o", str(out), *objs]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            print(_filter(r.stderr), file=sys.stderr)
            raise RuntimeError("link of libsiirl_hip.so failed")
        if verbose:
            print(f"[siirl_amd.build] linked {out}", flush=True)
    build_torch_layer(force=force or bool(jobs), verbose=verbose)
    return out


def build_torch_layer(force: bool = False, verbose: bool = True) -> Path:
    """``csrc/torch_ops.cpp`` -> ``lib/libsiirl_torch.so``: no device code, so the host compiler builds it; it links
    torch's own libraries and ``libsiirl_hip.so`` (found next to it through ``$ORIGIN``)."""
    import torch
    from torch.utils import cpp_extension as ce

    src = CSRC / "torch_ops.cpp"
    out = LIBDIR / TORCH_LIBNAME
    deps = [src, *(PKG.parent / "include").glob("*.h"), LIBDIR / LIBNAME]
    if not force and not _stale(out, deps):
        return out
    torch_lib = Path(torch.__file__).resolve().parent / "lib"
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    cmd = [CXX, "-O2", "-std=c++17", "-fPIC", "-shared", "-D__HIP_PLATFORM_AMD__", "-DUSE_ROCM",
           f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}", "-Wno-deprecated-declarations",
           *(f"-I{p}" for p in ce.include_paths()), f"-I{rocm}/include", str(src), "-o", str(out),
           f"-L{torch_lib}", "-ltorch", "-ltorch_cpu", "-lc10", "-lc10_hip", "-ltorch_hip",
           f"-L{LIBDIR}", "-lsiirl_hip", "-Wl,-rpath,$ORIGIN", "-Wl,--no-as-needed"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if verbose:
        print(f"[siirl_amd.build] {CXX} torch_ops.cpp: {'ok' if r.returncode == 0 else 'FAILED'}", flush=True)
    if r.returncode != 0:
        print(r.stderr, file=sys.stderr)
        raise RuntimeError("build of libsiirl_torch.so failed")
    return out


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--force", action="store_true")
    build(force=ap.parse_args().force)

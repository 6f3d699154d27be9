"""Builds ``siirl_amd/lib/libsiirl_hip.so`` from ``siirl_amd/csrc/*.hip`` with hipcc for gfx950.

Usage: ``python -m siirl_amd.build [--force]``.  The library is built in-tree so that it travels with
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

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
ARCH = "gfx950"
# -packed-fp32-ops: keep the compiler from forming v_pk_{add,mul,fma}_f32 out of scalar float code.
CXXFLAGS = ["-O3", "-std=c++17", "-fPIC", f"--offload-arch={ARCH}", "-Xclang", "-target-feature", "-Xclang",
            "-packed-fp32-ops", "-Wno-unused-command-line-argument", "-fno-gpu-rdc"]
# per-file additions: the numpy-emulating group statistics and the GAE recurrence must not be contracted into FMAs
EXTRA = {"group_ops.hip": ["-ffp-contract=off"], "gae.hip": ["-ffp-contract=off"],
         "reward.hip": ["-ffp-contract=off"]}


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
    return out


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--force", action="store_true")
    build(force=ap.parse_args().force)

"""Builds libmograd_hip.so (gfx950) from mograd_amd/csrc/*.hip with hipcc.

Usage: python -m mograd_amd.build [--force] [--jobs N]

Objects go to mograd_amd/csrc/build/, the library to mograd_amd/libmograd_hip.so.  A
source is recompiled when it or any header is newer than its object.
"""
from __future__ import annotations

import argparse
import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG = Path(__file__).resolve().parent
ROOT = PKG.parent
CSRC = PKG / "csrc"
OBJ_DIR = CSRC / "build"
LIB_PATH = PKG / "libmograd_hip.so"

ARCH = "gfx950"
# -packed-fp32-ops is switched off: v_pk_*_f32 forms are not to be generated.
HIPCC_FLAGS = [
    f"--offload-arch={ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fno-gpu-rdc",
    "-Wall",
    "-Wno-unused-function",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    f"-I{ROOT / 'include'}",
    f"-I{CSRC}",
]
# -z nodelete: a host that dlopens and later unloads the library must not unmap code that
# late destructors may still run (the hazard the reference's pin.c guards against,
# mograd/runtime/gpu/kernels/pin.c:14-21).
LINK_FLAGS = ["-shared", "-fPIC", f"--offload-arch={ARCH}", "-fno-gpu-rdc", "-Wl,-z,nodelete", "-Wl,--no-undefined"]


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and Path(cand).exists():
            return cand
    raise RuntimeError("hipcc not found; set HIPCC or install ROCm")


def _headers_mtime() -> float:
    hdrs = list(CSRC.glob("*.h")) + list((ROOT / "include").glob("*.h"))
    return max(h.stat().st_mtime for h in hdrs)


def _compile(hipcc: str, src: Path, obj: Path) -> tuple[Path, int, str]:
    cmd = [hipcc, *HIPCC_FLAGS, "-c", str(src), "-o", str(obj)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    # hipcc's host pass warns that it does not know the packed-fp32 feature: harmless.
    noise = ("is not a recognized feature for this target", "packed-fp32-ops")
    err = "\n".join(l for l in proc.stderr.splitlines() if not any(n in l for n in noise))
    return src, proc.returncode, err


def build(force: bool = False, jobs: int | None = None, verbose: bool = True) -> Path:
    hipcc = _hipcc()
    OBJ_DIR.mkdir(parents=True, exist_ok=True)
    sources = sorted(CSRC.glob("*.hip"))
    if not sources:
        raise RuntimeError(f"no sources under {CSRC}")
    hdr_time = _headers_mtime()
    todo = []
    objs = []
    for src in sources:
        obj = OBJ_DIR / (src.stem + ".o")
        objs.append(obj)
        if force or not obj.exists() or obj.stat().st_mtime < max(src.stat().st_mtime, hdr_time):
            todo.append((src, obj))
    jobs = jobs or min(8, os.cpu_count() or 1)
    if verbose and todo:
        print(f"[mograd_amd.build] compiling {len(todo)} file(s) for {ARCH} with {jobs} job(s)", flush=True)
    failed = []
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        for src, rc, err in pool.map(lambda so: _compile(hipcc, *so), todo):
            if err.strip() and verbose:
                print(f"--- {src.name}\n{err}", file=sys.stderr, flush=True)
            if rc != 0:
                failed.append(src.name)
    if failed:
        raise RuntimeError(f"hipcc failed for: {', '.join(failed)}")
    if todo or force or not LIB_PATH.exists():
        cmd = [hipcc, *LINK_FLAGS, *map(str, objs), "-o", str(LIB_PATH)]
        proc = subprocess.run(cmd, capture_output=True, text=True)
        if proc.returncode != 0:
            raise RuntimeError(f"link failed:\n{proc.stderr}")
        if verbose:
            print(f"[mograd_amd.build] linked {LIB_PATH}", flush=True)
    return LIB_PATH


def main() -> None:
    ap = argparse.ArgumentParser(description=__doc__)
    ap.add_argument("--force", action="store_true", help="recompile everything")
    ap.add_argument("--jobs", type=int, default=None)
    args = ap.parse_args()
    build(force=args.force, jobs=args.jobs)


if __name__ == "__main__":
    main()

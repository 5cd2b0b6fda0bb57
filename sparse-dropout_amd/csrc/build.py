"""Ahead-of-time build of libsparsedrop.so for gfx950 (MI355X) with hipcc.

    python sparse-dropout_amd/csrc/build.py [--force]

Every .hip file in this directory is one translation unit; they are compiled in parallel and linked
into flash_dropout/_lib/libsparsedrop.so next to the Python package, which loads it with ctypes.
hipcc cross-compiles for gfx950 without a GPU present.
"""
from __future__ import annotations

import argparse
import hashlib
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

CSRC = Path(__file__).resolve().parent
ROOT = CSRC.parent.parent
OUT_DIR = CSRC.parent / "flash_dropout" / "_lib"
OBJ_DIR = CSRC / "build"
LIB = OUT_DIR / "libsparsedrop.so"

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fvisibility=default",
    "-Wno-unused-command-line-argument",
    # keep the compiler from forming packed-fp32 VALU ops
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    f"-I{ROOT / 'include'}",
    f"-I{CSRC}",
    f"-I{OBJ_DIR}",
]


def sources() -> list[Path]:
    return sorted(CSRC.glob("*.hip"))


def source_hash() -> str:
    """Hash of everything the library is compiled from; the library reports the one it was built with
    (sd_source_hash) and the loader refuses a library whose sources have changed since."""
    h = hashlib.sha256()
    for f in [*sources(), *sorted(CSRC.glob("*.h")), *sorted((ROOT / "include").glob("*.h"))]:
        h.update(f.name.encode())
        h.update(f.read_bytes())
    return h.hexdigest()[:16]


def _stale(target: Path, deps: list[Path]) -> bool:
    if not target.exists():
        return True
    t = target.stat().st_mtime
    return any(d.stat().st_mtime > t for d in deps)


def _run(cmd: list[str]) -> None:
    proc = subprocess.run(cmd, capture_output=True, text=True)
    # hipcc's host pass warns that it does not know the packed-fp32 feature: harmless
    err = "\n".join(l for l in proc.stderr.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"command failed: {' '.join(cmd)}\n{proc.stdout}\n{err}")


def write_source_hash() -> Path:
    """(Re)writes the generated header api.hip includes; touched only when the hash changes."""
    OBJ_DIR.mkdir(parents=True, exist_ok=True)
    inc = OBJ_DIR / "source_hash.inc"
    line = f'#define SD_SOURCE_HASH "{source_hash()}"\n'
    if not inc.exists() or inc.read_text() != line:
        inc.write_text(line)  # newer than api.o: api.hip, which includes it, is recompiled by build()
    return inc


def build(force: bool = False, verbose: bool = False) -> Path:
    OUT_DIR.mkdir(parents=True, exist_ok=True)
    headers = sorted(CSRC.glob("*.h")) + sorted((ROOT / "include").glob("*.h"))
    headers.append(write_source_hash())
    jobs = []
    objs = []
    for src in sources():
        obj = OBJ_DIR / (src.stem + ".o")
        objs.append(obj)
        if force or _stale(obj, [src, *headers]):
            jobs.append([HIPCC, *FLAGS, "-c", str(src), "-o", str(obj)])
    if verbose:
        for j in jobs:
            print(" ".join(j), flush=True)
    with ThreadPoolExecutor(max_workers=min(8, max(1, len(jobs)))) as ex:
        list(ex.map(_run, jobs))
    if force or jobs or _stale(LIB, objs):
        _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(LIB), *map(str, objs)])
    return LIB


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--force", action="store_true")
    ap.add_argument("-v", "--verbose", action="store_true")
    a = ap.parse_args()
    print(build(a.force, a.verbose))

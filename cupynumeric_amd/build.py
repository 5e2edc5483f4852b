"""Build `libcpnsort.so` (HIP, gfx950) in-tree with hipcc.

    python -m cupynumeric_amd.build [--force] [--jobs N]

The translation units are compiled in parallel into `csrc/_obj/*.o` and linked into
`cupynumeric_amd/libcpnsort.so`.  No GPU is needed: hipcc cross-compiles for gfx950.
"""
from __future__ import annotations

import argparse
import concurrent.futures as cf
import os
import shutil
import subprocess
import sys
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
OBJ_DIR = CSRC / "_obj"
LIB_PATH = PKG_DIR / "libcpnsort.so"

SOURCES = [
    "sort_api.hip",
    "swapaxes.hip",
    "profile.hip",
    "convert.hip",
    "gather.hip",
    "searchsorted.hip",
    "unique.hip",
    "quantile.hip",
    "sort_keys8.hip",
    "sort_keys16.hip",
    "sort_keys32.hip",
    "sort_keys64.hip",
    "sort_keys128.hip",
]

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fno-gpu-rdc",
    "-Wall",
    "-Wno-unused-function",
    # packed fp32 instructions are kept out of every kernel of this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def hipcc_path() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not Path(exe).exists():
        raise RuntimeError("hipcc not found; a ROCm toolchain is required to build libcpnsort.so")
    return exe


def _headers_mtime() -> float:
    hdrs = list(CSRC.glob("*.h")) + [PKG_DIR.parent / "include" / "cpn_sort.h"]
    return max(h.stat().st_mtime for h in hdrs)


def _compile(src: str, force: bool, extra: list[str]) -> str:
    obj = OBJ_DIR / (Path(src).stem + ".o")
    src_path = CSRC / src
    if (
        not force
        and obj.exists()
        and obj.stat().st_mtime > src_path.stat().st_mtime
        and obj.stat().st_mtime > _headers_mtime()
    ):
        return str(obj)
    cmd = [hipcc_path(), *HIPCC_FLAGS, *extra, "-c", str(src_path), "-o", str(obj)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass warns that it does not know the packed-fp32 feature; that is harmless
    err = "\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return str(obj)


def build(force: bool = True, jobs: int | None = None, extra_flags: list[str] | None = None) -> Path:
    """Compile every translation unit and link the shared library.  Returns its path."""
    OBJ_DIR.mkdir(parents=True, exist_ok=True)
    jobs = jobs or min(len(SOURCES), os.cpu_count() or 4)
    extra = list(extra_flags or [])
    with cf.ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(lambda s: _compile(s, force, extra), SOURCES))
    cmd = [hipcc_path(), "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc", *objs, "-o", str(LIB_PATH)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stderr}")
    return LIB_PATH


def main() -> None:
    ap = argparse.ArgumentParser(description=__doc__)
    ap.add_argument("--force", action="store_true", help="recompile even if objects look current")
    ap.add_argument("--jobs", type=int, default=None)
    args = ap.parse_args()
    path = build(force=args.force, jobs=args.jobs)
    print(path)


if __name__ == "__main__":
    main()

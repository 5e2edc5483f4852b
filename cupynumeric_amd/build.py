"""Build `libcpnsort.so` (HIP, gfx950) in-tree with hipcc.

    python -m cupynumeric_amd.build [--force] [--jobs N]

The translation units are compiled in parallel into `csrc/_obj/*.o` and linked into
`cupynumeric_amd/libcpnsort.so`.  No GPU is needed: hipcc cross-compiles for gfx950.
"""
from __future__ import annotations

import argparse
import concurrent.futures as cf
import json
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
    # per-kernel registers, scratch and LDS as compiler remarks: collected into
    # csrc/_obj/<unit>.resources.json and checked below
    "-Rpass-analysis=kernel-resource-usage",
]

# Scratch memory (bytes per lane) a kernel may use.  The per-row kernels keep a whole row in
# registers; one that spills runs several times slower without failing any test (a 16-keys-per-
# thread shape once spilled 516 bytes per lane and took 3.3 ms instead of 0.8), so the build
# refuses it.  The scatter pass of the global sort is allowed the few words it is known to park.
SCRATCH_LIMITS = (("row_sort_kernel", 0), ("count16_", 0), ("onesweep_kernel", 32))


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
    lines = [l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l]
    resources, lines = _split_resource_remarks(lines)
    err = "\n".join(lines)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    (OBJ_DIR / (Path(src).stem + ".resources.json")).write_text(json.dumps(resources, indent=1))
    for kernel, use in resources.items():
        for pattern, limit in SCRATCH_LIMITS:
            if pattern in kernel and use.get("scratch_bytes_per_lane", 0) > limit:
                obj.unlink(missing_ok=True)
                raise RuntimeError(
                    f"{src}: kernel {kernel} spills {use['scratch_bytes_per_lane']} bytes per lane "
                    f"(limit {limit}); see SCRATCH_LIMITS in {Path(__file__).name}"
                )
    return str(obj)


_REMARK = "[-Rpass-analysis=kernel-resource-usage]"
_FIELDS = {
    "TotalSGPRs": "sgprs",
    "VGPRs": "vgprs",
    "ScratchSize [bytes/lane]": "scratch_bytes_per_lane",
    "Occupancy [waves/SIMD]": "waves_per_simd",
    "VGPRs Spill": "vgpr_spills",
    "LDS Size [bytes/block]": "lds_bytes",
}


def _split_resource_remarks(lines: list[str]) -> tuple[dict[str, dict[str, int]], list[str]]:
    """Take the compiler's per-kernel resource remarks (and the source excerpts printed under
    them) out of `lines`; returns ({mangled kernel name: figures}, the other lines)."""
    resources: dict[str, dict[str, int]] = {}
    rest: list[str] = []
    current: dict[str, int] | None = None
    skip = 0
    for line in lines:
        if _REMARK in line:
            text = line.split("remark:", 1)[1].replace(_REMARK, "").strip()
            key, _, value = text.partition(":")
            key, value = key.strip(), value.strip()
            if key == "Function Name":
                current = resources.setdefault(value, {})
            elif current is not None and key in _FIELDS and value.lstrip("-").isdigit():
                current[_FIELDS[key]] = int(value)
            skip = 2  # the quoted source line and its caret
        elif skip and (line.lstrip().startswith("|") or line.lstrip()[:1].isdigit()):
            skip -= 1
        elif line.startswith("In file included from") or "remarks generated" in line or "remark generated" in line:
            continue
        else:
            skip = 0
            rest.append(line)
    return resources, rest


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

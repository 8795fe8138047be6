"""Builds libbitsmoe_hip.so in-tree with hipcc for gfx950.

    python -m bitsmoe_amd.build                      # compile every .hip source and link
    python -m bitsmoe_amd.build forward_decode.hip   # recompile only the named sources, link with the other objects
    python -m bitsmoe_amd.build --timeline           # libbitsmoe_hip_timeline.so: the same library with in-kernel time
                                                     # stamps (python -m bitsmoe_amd.timeline reads them)

hipcc cross-compiles without a GPU, so this runs on a CPU-only host.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

CSRC = Path(__file__).resolve().parent / "csrc"
LIB_NAME = "libbitsmoe_hip.so"
LIB_PATH = CSRC / LIB_NAME

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Wall",
    "-Wno-unused-function",
    # packed-fp32 VALU forms are switched off for every HIP translation unit
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; libbitsmoe_hip.so cannot be built")
    return exe


def sources() -> list[Path]:
    return sorted(CSRC.glob("*.hip"))


def build_library(verbose: bool = True, jobs: int = 8, only: list[str] | None = None, timeline: bool = False) -> Path:
    """timeline=True: the variant with in-kernel time stamps (-DBITSMOE_TIMELINE), as libbitsmoe_hip_timeline.so."""
    hipcc = _hipcc()
    objdir = CSRC / ("build_timeline" if timeline else "build")
    lib_path = CSRC / ("libbitsmoe_hip_timeline.so" if timeline else LIB_NAME)
    objdir.mkdir(exist_ok=True)
    srcs = sources()
    # with `only`: also every source whose object is missing or older than a header (the objects share struct layouts)
    headers = [*CSRC.glob("*.h"), CSRC.parent.parent / "include" / "bitsmoe_hip.h"]
    newest_header = max(h.stat().st_mtime for h in headers if h.exists())

    def out_of_date(src: Path) -> bool:
        obj = objdir / (src.stem + ".o")
        return not obj.exists() or obj.stat().st_mtime < newest_header

    stale = [s for s in srcs if only and s.name not in only and out_of_date(s)]
    todo = [s for s in srcs if not only or s.name in only or s in stale]

    def compile_one(src: Path) -> Path:
        obj = objdir / (src.stem + ".o")
        extra = os.environ.get("BITSMOE_HIPCC_EXTRA", "").split()   # e.g. -DNAME for kernel experiments
        if timeline:
            extra.append("-DBITSMOE_TIMELINE")
        cmd = [hipcc, *HIPCC_FLAGS, *extra, "-c", str(src), "-o", str(obj)]
        if verbose:
            print("[bitsmoe build]", " ".join(cmd), flush=True)
        res = subprocess.run(cmd, capture_output=True, text=True)
        out = "\n".join(
            ln for ln in (res.stdout + res.stderr).splitlines()
            if "packed-fp32-ops" not in ln  # the host pass does not know the device feature
        )
        if res.returncode != 0:
            raise RuntimeError(f"hipcc failed for {src.name}:\n{out}")
        if verbose and out.strip():
            print(out, flush=True)
        return obj

    with ThreadPoolExecutor(max_workers=max(1, min(jobs, len(todo)))) as pool:
        list(pool.map(compile_one, todo))
    objs = [objdir / (s.stem + ".o") for s in srcs]
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(lib_path), *map(str, objs)]
    if verbose:
        print("[bitsmoe build]", " ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stdout}{res.stderr}")
    return lib_path


if __name__ == "__main__":
    args = [a for a in sys.argv[1:] if a != "--timeline"]
    path = build_library(only=args or None, timeline="--timeline" in sys.argv[1:])
    print(f"built {path}")
    sys.exit(0)

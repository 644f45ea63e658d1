"""Compile the HIP sources under csrc/ into flashsvd_amd/libflashsvd_hip.so (gfx950 only)."""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
LIB_PATH = PKG_DIR / "libflashsvd_hip.so"
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-value", "-Wno-unknown-attributes",
]


def sources() -> list[Path]:
    return sorted(CSRC.glob("*.hip"))


def build(verbose: bool = True, jobs: int = 8) -> Path:
    """Always recompiles every source; raises on the first compiler error."""
    objdir = CSRC / "build"
    objdir.mkdir(exist_ok=True)
    srcs = sources()
    if not srcs:
        raise RuntimeError(f"no HIP sources under {CSRC}")

    def compile_one(src: Path) -> Path:
        obj = objdir / (src.stem + ".o")
        cmd = [HIPCC, *FLAGS, "-c", str(src), "-o", str(obj)]
        res = subprocess.run(cmd, capture_output=True, text=True)
        if res.returncode != 0:
            raise RuntimeError(f"hipcc failed for {src.name}:\n{res.stdout}\n{res.stderr}")
        if verbose:
            warn = "\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l and l.strip())
            print(f"[build] {src.name} ok" + (f"\n{warn}" if warn else ""), flush=True)
        return obj

    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(compile_one, srcs))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc", *map(str, objs), "-o", str(LIB_PATH)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stdout}\n{res.stderr}")
    if verbose:
        print(f"[build] linked {LIB_PATH}", flush=True)
    return LIB_PATH


if __name__ == "__main__":
    build()
    sys.exit(0)

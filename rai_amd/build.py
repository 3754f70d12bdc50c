"""Builds librai_hip.so (gfx950) in-tree with hipcc.

Usage: python -m rai_amd.build [--force]
Each translation unit under rai_amd/csrc is compiled to an object in
rai_amd/csrc/build/ (in parallel) and linked into rai_amd/librai_hip.so.
"""
from __future__ import annotations

import concurrent.futures as cf
import os
import shutil
import subprocess
import sys
from pathlib import Path

PKG = Path(__file__).resolve().parent
ROOT = PKG.parent
CSRC = PKG / "csrc"
OBJ = CSRC / "build"
LIB = PKG / "librai_hip.so"

HIPCC = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"

# -packed-fp32-ops off: hipcc must not form v_pk_*_f32 from float code on this pool.
COMMON = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fno-gpu-rdc",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-result",
    f"-I{ROOT / 'include'}",
    f"-I{CSRC}",
]


# Per-file additions.  attention.hip: its MFMA accumulators are rescaled by ordinary vector instructions every
# key tile, so they must live in the registers those instructions can address; without this the compiler parks
# them in the accumulation registers and copies them out and back around every rescale.
EXTRA = {
    "attention.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"],
}


def sources() -> list[Path]:
    return sorted(list(CSRC.glob("*.hip")) + list(CSRC.glob("*.cpp")))


def _newer(a: Path, deps: list[Path]) -> bool:
    if not a.exists():
        return False
    t = a.stat().st_mtime
    return all(d.stat().st_mtime <= t for d in deps)


def _compile(src: Path, force: bool) -> Path:
    obj = OBJ / (src.name + ".o")
    headers = list(CSRC.glob("*.h")) + list((ROOT / "include").glob("*.h"))
    if not force and _newer(obj, [src] + headers):
        return obj
    cmd = [HIPCC, *COMMON, *EXTRA.get(src.name, []), "-x", "hip", "-c", str(src), "-o", str(obj)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src.name}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(force: bool = False, jobs: int | None = None) -> Path:
    OBJ.mkdir(parents=True, exist_ok=True)
    srcs = sources()
    if not srcs:
        raise RuntimeError("no sources under rai_amd/csrc")
    jobs = jobs or min(8, os.cpu_count() or 1)
    with cf.ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(lambda s: _compile(s, force), srcs))
    if force or not _newer(LIB, objs):
        cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc", "-o", str(LIB), *map(str, objs)]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"link failed:\n{r.stderr}")
    return LIB


if __name__ == "__main__":
    p = build(force="--force" in sys.argv)
    print(p)

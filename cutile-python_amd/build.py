"""Builds libmxgemm.so (HIP kernels + C ABI) for gfx950 with hipcc, in-tree.

    python cutile-python_amd/build.py [--force]

Each translation unit is compiled to an object file in parallel and the objects are linked into
cutile-python_amd/cutile_amd/libmxgemm.so.  hipcc cross-compiles: no GPU is needed to build.
"""
from __future__ import annotations

import argparse
import os
import pathlib
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

ROOT = pathlib.Path(__file__).resolve().parent
CSRC = ROOT / "csrc"
INCLUDE = ROOT.parent / "include"
OUT = ROOT / "cutile_amd" / "libmxgemm.so"
OBJ = ROOT / "build"
SOURCES = ["mx_api.hip", "mx_gemm_mfma.hip", "mx_gemm_pp.hip", "mx_gemm_pp32.hip", "mx_gemm_w4.hip", "mx_gemm_generic.hip", "mx_gemm_decode.hip", "mx_aux.hip", "mx_probe.hip"]
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         f"-I{INCLUDE}", f"-I{CSRC}", "-Wno-unused-command-line-argument"]
# Extra compiler flags for experiments (for example "-DSOMETHING=1"); objects built with a different flag set
# are never reused: the flag list is part of the up-to-date check (stamp file next to the objects).
FLAGS += os.environ.get("MXGEMM_EXTRA_FLAGS", "").split()


def _newer(src: pathlib.Path, obj: pathlib.Path) -> bool:
    if not obj.exists():
        return True
    deps = [src, *CSRC.glob("*.h"), INCLUDE / "mxgemm.h"]
    return any(d.stat().st_mtime > obj.stat().st_mtime for d in deps)


def _flags_changed() -> bool:
    """True when the objects on disk were built with other flags (the stamp is removed until the next build has
    compiled every object, so a failed build never leaves old objects looking current)."""
    stamp = OBJ / "flags.txt"
    if stamp.exists() and stamp.read_text() == " ".join(FLAGS):
        return False
    stamp.unlink(missing_ok=True)
    return True


def _compile(src: str, force: bool) -> pathlib.Path:
    s = CSRC / src
    o = OBJ / (s.stem + ".o")
    if force or _newer(s, o):
        cmd = ["hipcc", *FLAGS, "-c", str(s), "-o", str(o)]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed for {src}:\n{r.stdout}\n{r.stderr}")
    return o


def build(force: bool = False, jobs: int | None = None) -> pathlib.Path:
    OBJ.mkdir(exist_ok=True)
    force = _flags_changed() or force
    jobs = jobs or min(len(SOURCES), os.cpu_count() or 4, 8)
    with ThreadPoolExecutor(jobs) as ex:
        objs = list(ex.map(lambda s: _compile(s, force), SOURCES))
    (OBJ / "flags.txt").write_text(" ".join(FLAGS))
    cmd = ["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(OUT), *map(str, objs)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stdout}\n{r.stderr}")
    return OUT


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--force", action="store_true", help="recompile every translation unit")
    a = ap.parse_args()
    print(build(force=a.force))
    sys.exit(0)

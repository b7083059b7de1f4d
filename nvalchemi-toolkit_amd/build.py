"""Builds libnvalchemi_amd.so (the C-ABI library with the gfx950 kernels) in-tree with hipcc.

    python nvalchemi-toolkit_amd/build.py [--force] [--save-temps]

The library lands in nvalchemi-toolkit_amd/nvalchemi_amd/lib/ so that it travels with the
package; the Python side (nvalchemi_amd/_lib.py) loads it from there through ctypes.
"""

from __future__ import annotations

import argparse
import os
import subprocess
import sys
from pathlib import Path

HERE = Path(__file__).resolve().parent
CSRC = HERE / "csrc"
INCLUDE = HERE.parent / "include"
OUT_DIR = HERE / "nvalchemi_amd" / "lib"
LIB = OUT_DIR / "libnvalchemi_amd.so"
SOURCES = ["common.hip", "integrators.hip", "lj_pair.hip", "neighbor_list.hip", "coo.hip", "skin_wrap.hip", "observables.hip", "buffers.hip", "filter.hip", "langevin.hip", "nhc.hip", "f64.hip"]

FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fvisibility=hidden",
    "-fno-fast-math",
    "-munsafe-fp-atomics",
    # packed float32 VALU forms are kept out of generated code on this target
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wextra", "-Wno-unused-parameter", "-Wno-unknown-warning-option",
]


def hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (Path(cand).exists() or cand == "hipcc"):
            return cand
    raise RuntimeError("hipcc not found")


def build(force: bool = True, save_temps: bool = False, verbose: bool = False) -> Path:
    """Compile every HIP source for gfx950 and link the shared library."""
    OUT_DIR.mkdir(parents=True, exist_ok=True)
    obj_dir = HERE / "build"
    obj_dir.mkdir(exist_ok=True)
    srcs = [CSRC / s for s in SOURCES if (CSRC / s).exists()]
    deps = list(CSRC.glob("*.h")) + list(INCLUDE.glob("*.h"))
    newest_dep = max(p.stat().st_mtime for p in deps)
    objs = []
    procs = []
    for src in srcs:
        obj = obj_dir / (src.stem + ".o")
        objs.append(obj)
        if not force and obj.exists() and obj.stat().st_mtime > max(src.stat().st_mtime, newest_dep):
            continue
        cmd = [hipcc(), *FLAGS, f"-I{INCLUDE}", f"-I{CSRC}", "-c", str(src), "-o", str(obj)]
        if save_temps:
            cmd.insert(1, "--save-temps=obj")
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, cwd=obj_dir, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
    failed = False
    for src, p in procs:
        out, _ = p.communicate()
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l and l.strip())
        if p.returncode != 0:
            failed = True
            print(f"--- {src.name} FAILED\n{out}", file=sys.stderr)
        elif out and verbose:
            print(f"--- {src.name}\n{out}")
    if failed:
        raise RuntimeError("hipcc failed")
    cmd = [hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(LIB), *map(str, objs)]
    subprocess.run(cmd, check=True)
    return LIB


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--incremental", action="store_true", help="skip objects newer than their sources")
    ap.add_argument("--save-temps", action="store_true")
    ap.add_argument("-v", "--verbose", action="store_true")
    args = ap.parse_args()
    print(build(force=not args.incremental, save_temps=args.save_temps, verbose=args.verbose))

"""Build libsonicmoe_hip.so and libsonicmoe_hip_f16.so (gfx950) from csrc/*.hip with hipcc.  No torch headers, no
pybind: plain C ABI.  The two libraries come from the same sources and export the same entry points; the first takes
bf16 for the 16-bit tensors of the GEMM-side operators, the second (compiled with -DSMOE_ELEM_F16) fp16.

    python sonic-moe_amd/build.py [--verbose] [--resource-usage]

The libraries land in sonic-moe_amd/sonicmoe/lib/ so that they travel with the source tree.
"""

from __future__ import annotations

import argparse
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

ROOT = Path(__file__).resolve().parent
CSRC = ROOT / "csrc"
OUT_DIR = ROOT / "sonicmoe" / "lib"
OBJ_DIR = ROOT / "build"
LIB_NAME = "libsonicmoe_hip.so"
# (library, extra compiler flags, suffix of the object files)
VARIANTS = [(LIB_NAME, [], ""), ("libsonicmoe_hip_f16.so", ["-DSMOE_ELEM_F16"], "_f16")]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
ARCH = "gfx950"
FLAGS = [
    f"--offload-arch={ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Wall",
    "-Wno-unused-function",
    # keep the compiler from forming packed fp32 VALU ops out of scalar float code
    "-Xclang",
    "-target-feature",
    "-Xclang",
    "-packed-fp32-ops",
]


def _run(cmd: list[str], verbose: bool) -> str:
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    out = (res.stdout or "") + (res.stderr or "")
    # the host pass does not know the device-only target feature; drop that one harmless line
    out = "\n".join(l for l in out.splitlines() if "is not a recognized feature for this target" not in l)
    if res.returncode != 0:
        raise RuntimeError(f"command failed ({res.returncode}): {' '.join(cmd)}\n{out}")
    return out


def build(verbose: bool = False, resource_usage: bool = False, jobs: int | None = None) -> Path:
    sources = sorted(CSRC.glob("*.hip"))
    if not sources:
        raise RuntimeError(f"no sources under {CSRC}")
    OBJ_DIR.mkdir(parents=True, exist_ok=True)
    OUT_DIR.mkdir(parents=True, exist_ok=True)
    extra = ["-Rpass-analysis=kernel-resource-usage"] if resource_usage else []

    def compile_one(job: tuple[Path, list[str], str]) -> Path:
        src, defines, suffix = job
        obj = OBJ_DIR / (src.stem + suffix + ".o")
        out = _run([HIPCC, *FLAGS, *defines, *extra, "-c", str(src), "-o", str(obj)], verbose)
        if out.strip() and (verbose or resource_usage):
            print(out, flush=True)
        return obj

    # the longest compilations first: the wall time is the largest source's either way
    sources.sort(key=lambda p: -p.stat().st_size)
    work = [(src, defines, suffix) for src in sources for _, defines, suffix in VARIANTS]
    jobs = jobs or min(len(work), os.cpu_count() or 1, 8)
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(compile_one, work))
    for name, _, suffix in VARIANTS:
        mine = [o for o, (_, _, sfx) in zip(objs, work) if sfx == suffix]
        tmp = OUT_DIR / (name + ".tmp")
        # -Bsymbolic: the two libraries define the same symbols; each binds its internal references (kernel stubs
        # included) to its own definitions even if a host program loads the other one with RTLD_GLOBAL first
        _run([HIPCC, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-Wl,-Bsymbolic", "-o", str(tmp), *map(str, mine)],
             verbose)
        os.replace(tmp, OUT_DIR / name)
    return OUT_DIR / LIB_NAME


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--verbose", action="store_true")
    ap.add_argument("--resource-usage", action="store_true", help="print per-kernel register / LDS / occupancy remarks")
    ap.add_argument("-j", "--jobs", type=int, default=None)
    a = ap.parse_args()
    try:
        print(build(a.verbose, a.resource_usage, a.jobs))
    except RuntimeError as e:
        print(e, file=sys.stderr)
        sys.exit(1)

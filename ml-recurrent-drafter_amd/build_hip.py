"""Builds libredrafter_hip.so (the C-ABI library) from csrc/ with hipcc for gfx950.

    python ml-recurrent-drafter_amd/build_hip.py          # compile everything, link in-tree

The shared object is written next to the Python package so that it travels with the source tree;
no JIT cache is involved.  Cross-compiles without a GPU.
"""

from __future__ import annotations

import concurrent.futures
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(CSRC, "obj")
LIB = os.path.join(HERE, "recurrent_drafting_amd", "libredrafter_hip.so")
# measurement yardsticks that kernel_bench.py loads: a shared object of their own, outside the C ABI
BENCH_CSRC = os.path.join(HERE, "bench_csrc")
BENCH_LIB = os.path.join(BENCH_CSRC, "libredrafter_bench.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fvisibility=hidden",
    "-DNDEBUG",
    # packed-FP32 VALU forms are kept out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    "-I", os.path.join(ROOT, "include"),
    "-I", CSRC,
]


def sources() -> list[str]:
    return sorted(
        os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith((".hip", ".cpp"))
    )


def bench_sources() -> list[str]:
    return sorted(os.path.join(BENCH_CSRC, f) for f in os.listdir(BENCH_CSRC) if f.endswith(".hip"))


def _compile(src: str) -> str:
    obj = os.path.join(OBJ, os.path.basename(src) + ".o")
    cmd = [HIPCC, *FLAGS, "-c", src, "-o", obj]
    if src.endswith(".hip"):
        cmd[1:1] = ["-x", "hip"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{r.stdout}\n{r.stderr}")
    noise = "is not a recognized feature for this target"
    warn = "\n".join(line for line in r.stderr.splitlines() if line.strip() and noise not in line)
    if warn.strip():
        sys.stderr.write(warn + "\n")
    return obj


def build(jobs: int | None = None, verbose: bool = True) -> str:
    os.makedirs(OBJ, exist_ok=True)
    srcs, bench_srcs = sources(), bench_sources()
    jobs = jobs or min(len(srcs) + len(bench_srcs), 8)
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as ex:
        all_objs = list(ex.map(_compile, srcs + bench_srcs))
    objs, bench_objs = all_objs[: len(srcs)], all_objs[len(srcs):]
    for lib, group in ((LIB, objs), (BENCH_LIB, bench_objs)):
        cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", lib, *group]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"link failed:\n{r.stdout}\n{r.stderr}")
    if verbose:
        print(f"built {LIB} from {len(srcs)} sources and {BENCH_LIB} from {len(bench_srcs)}")
    return LIB


if __name__ == "__main__":
    build()

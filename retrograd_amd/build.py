"""Builds libretro_hip.so (the C-ABI library) for gfx950 with hipcc.

The library is compiled in-tree (retrograd_amd/lib/) so it travels with the
source tree; nothing is installed into site-packages.
"""

from __future__ import annotations

import os
import subprocess
import sys
from pathlib import Path

PKG = Path(__file__).resolve().parent
CSRC = PKG / "csrc"
LIB_DIR = PKG / "lib"
LIB_PATH = LIB_DIR / "libretro_hip.so"
SOURCES = ["kernels.hip", "mm_lds.hip", "gemv.hip", "moe.hip", "mxfp4_scaled.hip", "engine.cpp", "generate.cpp", "capi.cpp", "capi_trainer.cpp", "capi_test.cpp"]
# host-only sources (the step scheduler): plain C++, no device pass
HOST_SOURCES = ["sched/prefix_tree.cpp", "sched/scheduler.cpp", "sched/fake_backend.cpp", "sched/engine_backend.cpp",
                "sched/capi_sched.cpp"]
HOST_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-Wall", "-Wextra", "-Wno-unused-parameter", "-D__HIP_PLATFORM_AMD__",
              "-I/opt/rocm/include"]
HEADERS = ["kernels.hpp", "dev_common.hpp", "engine.hpp", "sampler.hpp", "gguf_file.hpp"]

# packed-fp32 code generation is switched off for every HIP translation unit.
HIP_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wextra",
             "-Wno-unused-parameter", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    raise RuntimeError("hipcc not found")


def _compile(cmd, src, verbose):
    if verbose:
        print(" ".join(cmd), file=sys.stderr)
    res = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in res.stderr.splitlines() if noise not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed on %s:\n%s" % (src, err))
    if verbose and err.strip():
        print(err, file=sys.stderr)


def build(verbose: bool = False, incremental: bool = False) -> Path:
    """Compiles every source (several at a time) and links the library. `incremental` skips a source whose object
    is newer than it and than every header; the default recompiles everything."""
    from concurrent.futures import ThreadPoolExecutor

    LIB_DIR.mkdir(exist_ok=True)
    obj_dir = LIB_DIR / "obj"
    obj_dir.mkdir(exist_ok=True)
    headers = [p for p in CSRC.rglob("*.h*")] + list((PKG.parent / "include").glob("*.h"))
    newest_header = max(p.stat().st_mtime for p in headers)
    jobs, objs = [], []
    for src in SOURCES + HOST_SOURCES:
        host = src in HOST_SOURCES
        obj = obj_dir / (src.replace("/", "_").rsplit(".", 1)[0] + ".o")
        objs.append(str(obj))
        if incremental and obj.exists() and obj.stat().st_mtime > max((CSRC / src).stat().st_mtime, newest_header):
            continue
        if host:
            cmd = [hipcc(), *HOST_FLAGS, "-x", "c++", "-c", str(CSRC / src), "-o", str(obj)]
        else:
            cmd = [hipcc(), *HIP_FLAGS, "-x", "hip", "-c", str(CSRC / src), "-o", str(obj)]
        jobs.append((cmd, src))
    with ThreadPoolExecutor(max_workers=min(8, os.cpu_count() or 1)) as pool:
        for f in [pool.submit(_compile, cmd, src, verbose) for cmd, src in jobs]:
            f.result()
    cmd = [hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(LIB_PATH), *objs]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("link failed:\n" + res.stderr)
    # the stand-alone micro-benchmark of the compute unit's issue and LDS rates (no part of the library)
    ub_src, ub_bin = CSRC / "ubench" / "issue_model.hip", LIB_DIR / "ubench_issue_model"
    if not (incremental and ub_bin.exists() and ub_bin.stat().st_mtime > ub_src.stat().st_mtime):
        _compile([hipcc(), *[f for f in HIP_FLAGS if f != "-fPIC"], "-o", str(ub_bin), str(ub_src)], "ubench/issue_model.hip", verbose)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose=True, incremental="--incremental" in sys.argv))

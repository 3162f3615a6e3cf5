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
SOURCES = ["kernels.hip", "mm_lds.hip", "moe.hip", "engine.cpp", "generate.cpp", "capi.cpp", "capi_trainer.cpp", "capi_test.cpp"]
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


def build(verbose: bool = False) -> Path:
    LIB_DIR.mkdir(exist_ok=True)
    obj_dir = LIB_DIR / "obj"
    obj_dir.mkdir(exist_ok=True)
    objs = []
    for src in SOURCES:
        obj = obj_dir / (src.rsplit(".", 1)[0] + ".o")
        cmd = [hipcc(), *HIP_FLAGS, "-x", "hip", "-c", str(CSRC / src), "-o", str(obj)]
        if verbose:
            print(" ".join(cmd), file=sys.stderr)
        res = subprocess.run(cmd, capture_output=True, text=True)
        noise = "is not a recognized feature for this target"
        err = "\n".join(l for l in res.stderr.splitlines() if noise not in l)
        if res.returncode != 0:
            raise RuntimeError("hipcc failed on %s:\n%s" % (src, err))
        if verbose and err.strip():
            print(err, file=sys.stderr)
        objs.append(str(obj))
    for src in HOST_SOURCES:
        obj = obj_dir / (src.replace("/", "_").rsplit(".", 1)[0] + ".o")
        cmd = [hipcc(), *HOST_FLAGS, "-x", "c++", "-c", str(CSRC / src), "-o", str(obj)]
        if verbose:
            print(" ".join(cmd), file=sys.stderr)
        res = subprocess.run(cmd, capture_output=True, text=True)
        if res.returncode != 0:
            raise RuntimeError("hipcc failed on %s:\n%s" % (src, res.stderr))
        if verbose and res.stderr.strip():
            print(res.stderr, file=sys.stderr)
        objs.append(str(obj))
    cmd = [hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(LIB_PATH), *objs]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("link failed:\n" + res.stderr)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose=True))

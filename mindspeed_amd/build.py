"""Build recipe for libmindspeed_amd.so (hipcc, gfx950 only, in-tree).

``python -m mindspeed_amd.build`` compiles every ``csrc/*.hip`` translation
unit for gfx950 and links them into ``mindspeed_amd/libmindspeed_amd.so``.
hipcc cross-compiles, so this works on a host without a GPU.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(HERE, "build")
LIB_PATH = os.path.join(HERE, "libmindspeed_amd.so")
TRACE_LIB_PATH = os.path.join(HERE, "libmindspeed_amd_trace.so")   # diagnostic variant: per-tile time stamps
MICROBENCH_CSRC = os.path.join(HERE, "csrc_microbench")
MICROBENCH_LIB_PATH = os.path.join(HERE, "libmindspeed_amd_microbench.so")   # measurement helpers (plain copy kernel)

ARCH = "gfx950"
# packed-fp32 VALU forms are switched off for every device translation unit.
HIPCC_FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-fPIC", "-std=c++17",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found: the MI355X kernels cannot be built")
    return exe


def sources():
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def source_hash() -> str:
    """First 16 hex digits of the SHA-256 over the kernel sources (csrc/*.hip, csrc/*.h, the C-ABI header) in name
    order: names the build that measured figures (profiles/*.json) belong to."""
    import hashlib

    h = hashlib.sha256()
    files = sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith((".hip", ".h")))
    files.append(os.path.join(HERE, "..", "include", "mindspeed_amd.h"))
    for f in files:
        h.update(os.path.basename(f).encode())
        with open(f, "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()[:16]


def _compile(src: str, force: bool, extra=(), suffix="") -> str:
    obj = os.path.join(OBJ_DIR, os.path.basename(src)[:-4] + suffix + ".o")
    deps = [src, os.path.join(HERE, "..", "include", "mindspeed_amd.h")]
    deps += [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")]
    if not force and os.path.exists(obj) and all(os.path.getmtime(obj) > os.path.getmtime(d) for d in deps):
        return obj
    cmd = [_hipcc(), *HIPCC_FLAGS, *extra, "-c", src, "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{res.stderr}")
    return obj


def build(force: bool = True, verbose: bool = False) -> str:
    """Compile and link the library; returns its path."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    srcs = sources()
    with ThreadPoolExecutor(max_workers=min(8, len(srcs))) as pool:
        objs = list(pool.map(lambda s: _compile(s, force), srcs))
    cmd = [_hipcc(), f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", LIB_PATH, *objs]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stderr}")
    if verbose:
        print(f"built {LIB_PATH} from {len(srcs)} translation units")
    return LIB_PATH


def build_trace(verbose: bool = False) -> str:
    """The diagnostic variant of the library: the grouped-matmul fast kernels compiled with MS_TRACE_TILES (every
    workgroup records time stamps of its phases, read back with ms_trace_read; see profile_tools timeline).  Not
    loaded by anything else; select it with MINDSPEED_AMD_LIB."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    objs = [_compile(s, True, ("-DMS_TRACE_TILES",), "_trace") if s.endswith("gmm_fast.hip") else _compile(s, False)
            for s in sources()]
    cmd = [_hipcc(), f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", TRACE_LIB_PATH, *objs]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stderr}")
    if verbose:
        print(f"built {TRACE_LIB_PATH}")
    return TRACE_LIB_PATH


def build_microbench(verbose: bool = False) -> str:
    """The measurement helpers (csrc_microbench/*.hip: the plain copy kernel the microbenchmarks and the counter
    calibration use).  A library of its own: nothing in it is part of the product's C ABI."""
    srcs = sorted(os.path.join(MICROBENCH_CSRC, f) for f in os.listdir(MICROBENCH_CSRC) if f.endswith(".hip"))
    cmd = [_hipcc(), *HIPCC_FLAGS, "-shared", "-o", MICROBENCH_LIB_PATH, *srcs]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed for the microbench helpers:\n{res.stderr}")
    if verbose:
        print(f"built {MICROBENCH_LIB_PATH}")
    return MICROBENCH_LIB_PATH


if __name__ == "__main__":
    if "--trace" in sys.argv:
        build_trace(verbose=True)
    elif "--microbench" in sys.argv:
        build_microbench(verbose=True)
    else:
        build(force="--incremental" not in sys.argv, verbose=True)

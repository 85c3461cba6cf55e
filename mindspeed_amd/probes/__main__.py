from __future__ import annotations

import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
BIN = os.path.join(HERE, "bin")
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wno-unused-command-line-argument", "-pthread"]


def names():
    return sorted(f[:-4] for f in os.listdir(HERE) if f.endswith(".hip"))


def build(name: str) -> str:
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    os.makedirs(BIN, exist_ok=True)
    exe = os.path.join(BIN, name)
    res = subprocess.run([hipcc, *FLAGS, os.path.join(HERE, name + ".hip"), "-o", exe], capture_output=True, text=True)
    if res.returncode != 0:
        raise SystemExit(f"hipcc failed for {name}:\n{res.stderr}")
    return exe


def main(argv):
    if len(argv) >= 1 and argv[0] == "build":
        for n in (argv[1:] or names()):
            print("built", build(n))
        return 0
    if len(argv) == 2 and argv[0] == "run" and argv[1] in names():
        exe = os.path.join(BIN, argv[1])
        if not os.path.exists(exe):
            build(argv[1])
        return subprocess.run([exe]).returncode
    print(__import__("mindspeed_amd.probes").probes.__doc__)
    print("probes:", ", ".join(names()))
    return 2


if __name__ == "__main__":
    sys.exit(main(sys.argv[1:]))

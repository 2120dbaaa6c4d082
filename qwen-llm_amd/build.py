"""Builds libdflash_hip.so (hand-written HIP for gfx950) in-tree with hipcc."""
from __future__ import annotations

import glob
import os
import subprocess
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
LIB_PATH = os.path.join(PKG_DIR, "libdflash_hip.so")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-fno-gpu-rdc",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def sources():
    return sorted(glob.glob(os.path.join(CSRC, "*.hip")))


def is_stale() -> bool:
    if not os.path.exists(LIB_PATH):
        return True
    t = os.path.getmtime(LIB_PATH)
    deps = sources() + glob.glob(os.path.join(CSRC, "*.h")) + \
        glob.glob(os.path.join(PKG_DIR, "..", "include", "*.h"))
    return any(os.path.getmtime(d) > t for d in deps)


def build(verbose: bool = False) -> str:
    """Compile every HIP source into one shared library; always recompiles."""
    objs = []
    procs = []
    for src in sources():
        obj = src[:-4] + ".o"
        cmd = [HIPCC] + [f for f in FLAGS if f != "-shared"] + ["-c", src, "-o", obj]
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs.append(obj)
    failed = False
    for src, p in procs:
        out, _ = p.communicate()
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l)
        if p.returncode != 0:
            failed = True
            sys.stderr.write(f"hipcc failed for {src}:\n{out}\n")
        elif verbose and out.strip():
            sys.stderr.write(out + "\n")
    if failed:
        raise RuntimeError("hipcc compilation failed")
    link = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc", "-o", LIB_PATH] + objs
    r = subprocess.run(link, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        sys.stderr.write(r.stdout)
        raise RuntimeError("hipcc link failed")
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose=True))

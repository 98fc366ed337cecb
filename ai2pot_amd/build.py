"""Build recipe of libai2pot_hip.so (gfx950) and of the operator bind libraries.

    python -m ai2pot_amd.build            # HIP library only
    python -m ai2pot_amd.build --bind     # plus the torch / CPython bind libraries

hipcc cross-compiles without a GPU.  Everything is built in-tree, next to the sources.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libai2pot_hip.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    # packed-FP32 instruction selection is switched off for all device code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-result", "-Wno-unknown-warning-option",
]
# translation units whose arithmetic must match the reference's x86-64 build bit for bit
# (no fused multiply-add contraction)
NO_CONTRACT = {"nblist.hip"}


def hip_sources():
    return sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))


def _compile(src):
    obj = os.path.join(CSRC, src[:-4] + ".o")
    flags = list(HIP_FLAGS)
    if src in NO_CONTRACT:
        flags.append("-ffp-contract=off")
    cmd = [HIPCC] + flags + ["-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s\n%s" % (src, " ".join(cmd), r.stderr[-8000:]))
    warn = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l and l.strip())
    return obj, warn


def build_hip(verbose=True, jobs=8):
    srcs = hip_sources()
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        results = list(ex.map(_compile, srcs))
    objs = [o for o, _ in results]
    if verbose:
        for (_, w), s in zip(results, srcs):
            if w:
                print("[%s]\n%s" % (s, w))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n%s" % r.stderr[-4000:])
    for o in objs:
        os.remove(o)
    if verbose:
        print("built", LIB)
    return LIB


if __name__ == "__main__":
    build_hip()
    if "--bind" in sys.argv:
        from ai2pot_amd import bind_build
        bind_build.build_bind()

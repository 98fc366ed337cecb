"""Builds the drop-in operator libraries into ai2pot_amd/_lib/ (the directory a reference
installation calls ai2pot/_lib):

    libnep_bind.so, libmtpr_bind.so, libnnmtp_bind.so, libfvt_sr_op_bind.so, libnblist_bind.so   -- TORCH_LIBRARY registrations
    nblist.<abi>.so                                          -- CPython module `nblist`

They are thin: argument checks plus calls into libai2pot_hip.so (found through an $ORIGIN
rpath one directory up).  Host C++ only; compiled with g++ against the torch headers.
"""
import os
import subprocess
import sysconfig
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "csrc", "bind")
OUT = os.path.join(HERE, "_lib")
CXX = os.environ.get("CXX", "g++")
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")


def _torch_flags():
    import torch
    from torch.utils import cpp_extension as ce
    inc = ["-I" + p for p in ce.include_paths()]
    libdir = os.path.join(os.path.dirname(torch.__file__), "lib")
    abi = "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI)
    return inc, libdir, abi


def _run(cmd):
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("build failed:\n%s\n%s" % (" ".join(cmd), r.stderr[-6000:]))


def _torch_lib(name):
    inc, libdir, abi = _torch_flags()
    py_inc = "-I" + sysconfig.get_paths()["include"]
    out = os.path.join(OUT, "lib%s.so" % name)
    cmd = [CXX, "-std=c++17", "-O2", "-fPIC", "-shared", "-w", abi, "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           "-I" + os.path.join(ROCM, "include"), py_inc] + inc + [
           os.path.join(SRC, name + ".cc"), "-o", out,
           "-L" + HERE, "-lai2pot_hip", "-L" + libdir, "-ltorch", "-ltorch_cpu", "-ltorch_hip", "-lc10", "-lc10_hip", "-lamdhip64",
           "-Wl,-rpath,$ORIGIN/..", "-Wl,-rpath," + libdir]
    _run(cmd)
    return out


def _nblist_module():
    import numpy
    ext = sysconfig.get_config_var("EXT_SUFFIX")
    out = os.path.join(OUT, "nblist" + ext)
    cmd = [CXX, "-std=c++17", "-O2", "-fPIC", "-shared", "-w", "-D__HIP_PLATFORM_AMD__=1",
           "-I" + os.path.join(ROCM, "include"), "-I" + sysconfig.get_paths()["include"],
           "-I" + numpy.get_include(), os.path.join(SRC, "nblist_module.cc"), "-o", out,
           "-L" + HERE, "-lai2pot_hip", "-L" + os.path.join(ROCM, "lib"), "-lamdhip64",
           "-Wl,-rpath,$ORIGIN/..", "-Wl,-rpath," + os.path.join(ROCM, "lib")]
    _run(cmd)
    return out


def build_bind(verbose=True):
    if not os.path.exists(os.path.join(HERE, "libai2pot_hip.so")):
        raise RuntimeError("build libai2pot_hip.so first (python -m ai2pot_amd.build)")
    os.makedirs(OUT, exist_ok=True)
    jobs = [lambda: _torch_lib("nep_bind"), lambda: _torch_lib("mtpr_bind"), lambda: _torch_lib("nnmtp_bind"),
            lambda: _torch_lib("fvt_sr_op_bind"), lambda: _torch_lib("nblist_bind"), _nblist_module]
    with ThreadPoolExecutor(max_workers=6) as ex:
        outs = [f.result() for f in [ex.submit(j) for j in jobs]]
    if verbose:
        for o in outs:
            print("built", o)
    return outs


if __name__ == "__main__":
    build_bind()

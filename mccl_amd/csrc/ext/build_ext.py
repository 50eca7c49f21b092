"""Compiles the torch extension ``mccl_amd/_C*.so`` in-tree with g++ (host code
only: every kernel lives in ``libmccl_hip.so``)."""
from __future__ import annotations

import concurrent.futures as cf
import os
import subprocess
import sysconfig

HERE = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.dirname(os.path.dirname(HERE))
OBJ = os.path.join(PKG, "build", "ext")
SOURCES = ["HipKernels.cpp", "Compression.cpp", "RingDriver.cpp", "Registration.cpp"]


def target() -> str:
    return os.path.join(PKG, "_C" + sysconfig.get_config_var("EXT_SUFFIX"))


def _run(cmd):
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if p.returncode != 0:
        raise RuntimeError("command failed: " + " ".join(cmd) + "\n" + p.stdout)
    if p.stdout.strip():
        print(p.stdout)


def build(force: bool = True) -> str:
    import torch
    from torch.utils import cpp_extension as ce

    os.makedirs(OBJ, exist_ok=True)
    tdir = os.path.dirname(torch.__file__)
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    inc = [f"-I{p}" for p in ce.include_paths()] + [f"-I{rocm}/include", f"-I{sysconfig.get_paths()['include']}"]
    flags = ["-std=c++17", "-O2", "-fPIC", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
             "-DTORCH_EXTENSION_NAME=_C", "-DTORCH_API_INCLUDE_EXTENSION_H",
             f"-D_GLIBCXX_USE_CXX11_ABI={int(torch.compiled_with_cxx11_abi())}", "-Wno-deprecated-declarations", "-Wno-attributes", "-fvisibility=hidden"]
    cxx = os.environ.get("CXX", "g++")
    objs, jobs = [], []
    for s in SOURCES:
        o = os.path.join(OBJ, s.replace(".cpp", ".o"))
        objs.append(o)
        jobs.append([cxx, *flags, *inc, "-c", os.path.join(HERE, s), "-o", o])
    with cf.ThreadPoolExecutor(max_workers=4) as ex:
        list(ex.map(_run, jobs))
    out = target()
    _run([cxx, "-shared", "-o", out, *objs, f"-L{PKG}", "-lmccl_hip", f"-L{tdir}/lib", "-lc10", "-lc10_hip",
          "-ltorch_cpu", "-ltorch_hip", "-ltorch", "-ltorch_python", "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{tdir}/lib"])
    return out

"""Builds the native pieces in-tree.

``libmccl_hip.so``  the gfx950 kernels behind the C ABI of ``include/mccl_hip.h``
                    (hipcc, no torch dependency)
``_C*.so``          the torch extension mirroring the reference's C++ / pybind
                    surface on top of that C ABI (see ``csrc/ext``)

Run ``python -m mccl_amd.build`` (both), or ``--lib`` / ``--ext``.
"""
from __future__ import annotations

import argparse
import concurrent.futures as cf
import os
import subprocess
import sys
import sysconfig

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libmccl_hip.so")

HIP_SOURCES = ["runtime.hip", "fold.hip", "topk.hip", "sparse.hip", "cast.hip"]

# -ffp-contract=off: every fold is one IEEE operation per element, never an FMA.
# packed-fp32-ops is switched off for all device code.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    "-fno-fast-math", "-Wall", "-Wno-unused-function", "-Wno-pass-failed",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def _run(cmd):
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in p.stdout.splitlines()
                    if "packed-fp32-ops' is not a recognized feature" not in l)
    if p.returncode != 0:
        raise RuntimeError("command failed: " + " ".join(cmd) + "\n" + out)
    if out.strip():
        print(out)


def build_lib(force: bool = True) -> str:
    os.makedirs(OBJ, exist_ok=True)
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    objs = []
    jobs = []
    for src in HIP_SOURCES:
        s = os.path.join(CSRC, src)
        o = os.path.join(OBJ, src.replace(".hip", ".o"))
        objs.append(o)
        jobs.append([hipcc, *HIPCC_FLAGS, "-c", s, "-o", o])
    with cf.ThreadPoolExecutor(max_workers=5) as ex:
        list(ex.map(_run, jobs))
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs])
    return LIB


def build_ext(force: bool = True) -> str:
    from mccl_amd.csrc.ext import build_ext as _b  # noqa: WPS433
    return _b.build(force=force)


def main(argv=None) -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--lib", action="store_true")
    ap.add_argument("--ext", action="store_true")
    a = ap.parse_args(argv)
    both = not (a.lib or a.ext)
    if a.lib or both:
        print("built", build_lib())
    if a.ext or both:
        print("built", build_ext())
    return 0


if __name__ == "__main__":
    sys.exit(main())

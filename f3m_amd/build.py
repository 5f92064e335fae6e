"""Builds the gfx950 shared library of the engine with hipcc (cross-compiles without a GPU).

    python -m f3m_amd.build            # -> f3m_amd/lib/libf3m.so
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
LIB = os.path.join(LIBDIR, "libf3m.so")

COMMON = ["--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17", "-Wall", "-Wno-unused-result",
          # packed fp32 arithmetic is kept off: the compiler must not form v_pk_*_f32 from scalar code
          "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
UNITS = [
    # box division and lists: every fp32 operation rounds once, division and sqrt correctly rounded
    ("f3m_geom.hip", ["-ffp-contract=off", "-fhip-fp32-correctly-rounded-divide-sqrt"]),
    ("f3m_field.hip", []),
    ("f3m_plan.hip", []),
]


def build(verbose=True, hipcc=None):
    hipcc = hipcc or os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    os.makedirs(LIBDIR, exist_ok=True)
    objs = []
    for src, extra in UNITS:
        obj = os.path.join(LIBDIR, src.replace(".hip", ".o"))
        cmd = [hipcc] + COMMON + extra + ["-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        subprocess.check_call(cmd)
        objs.append(obj)
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return LIB


if __name__ == "__main__":
    build()
    sys.exit(0)

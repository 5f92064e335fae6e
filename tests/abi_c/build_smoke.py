"""Compiles tests/abi_c/abi_smoke.c (plain C, HIP runtime API only) against include/f3m.h and the engine library.

    python tests/abi_c/build_smoke.py        # -> tests/abi_c/_build/abi_smoke
"""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
OUT = os.path.join(HERE, "_build", "abi_smoke")


def build(verbose=True):
    os.makedirs(os.path.dirname(OUT), exist_ok=True)
    libdir = os.path.join(ROOT, "f3m_amd", "lib")
    cmd = ["gcc", "-std=c11", "-O2", "-Wall", "-D__HIP_PLATFORM_AMD__", "-I/opt/rocm/include", "-I" + os.path.join(ROOT, "include"),
           os.path.join(HERE, "abi_smoke.c"), "-o", OUT, "-L" + libdir, "-lf3m", "-L/opt/rocm/lib", "-lamdhip64", "-lm",
           "-Wl,-rpath,$ORIGIN/../../../f3m_amd/lib", "-Wl,-rpath,/opt/rocm/lib"]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return OUT


if __name__ == "__main__":
    build()

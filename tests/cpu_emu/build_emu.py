"""TEST INFRASTRUCTURE: compiles the engine's kernel sources for the CPU with g++ against
tests/cpu_emu/hip_emu.h, so `-m "not gpu"` tests can run the real kernel logic on tiny inputs.
The result (tests/cpu_emu/_build/libf3m_emu.so) is never loaded by the f3m_amd package."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
CSRC = os.path.join(ROOT, "f3m_amd", "csrc")
OUT = os.path.join(HERE, "_build", "libf3m_emu.so")
SRCS = ["f3m_geom.hip", "f3m_field.hip", "f3m_plan.hip"]


def build(force=False, sanitize=False):
    srcs = [os.path.join(CSRC, s) for s in SRCS]
    deps = srcs + [os.path.join(CSRC, h) for h in ("f3m_rt.h", "f3m_engine.h")] + [os.path.join(HERE, "hip_emu.h"),
                                                                                    os.path.join(ROOT, "include", "f3m.h")]
    if not force and os.path.exists(OUT) and all(os.path.getmtime(OUT) > os.path.getmtime(p) for p in deps):
        return OUT
    os.makedirs(os.path.dirname(OUT), exist_ok=True)
    objs = []
    for s in srcs:
        o = os.path.join(HERE, "_build", os.path.basename(s) + ".o")
        flags = ["-O1", "-g", "-fPIC", "-std=c++17", "-DF3M_CPU_EMU", "-I", HERE, "-I", CSRC, "-Wall", "-Wno-unused",
                 "-Wno-unknown-pragmas", "-Wno-maybe-uninitialized"]
        if s.endswith("f3m_geom.hip"):
            flags += ["-ffp-contract=off"]
        if sanitize:
            flags += ["-fsanitize=address,undefined", "-fno-omit-frame-pointer"]
        subprocess.check_call(["g++"] + flags + ["-x", "c++", "-c", s, "-o", o])
        objs.append(o)
    link = ["g++", "-shared", "-o", OUT] + objs
    if sanitize:
        link += ["-fsanitize=address,undefined"]
    subprocess.check_call(link)
    return OUT


def build_sanitize_driver():
    """tests/cpu_emu/sanitize_driver.cpp and the kernel sources in one executable under AddressSanitizer and
    UndefinedBehaviorSanitizer (an executable, so that the sanitizer runtime comes first without preloading anything).
    Takes a minute or two to compile."""
    out = os.path.join(HERE, "_build", "sanitize_driver")
    srcs = [os.path.join(CSRC, s) for s in SRCS]
    os.makedirs(os.path.dirname(out), exist_ok=True)
    flags = ["-O1", "-g", "-std=c++17", "-DF3M_CPU_EMU", "-fsanitize=address,undefined", "-fno-omit-frame-pointer",
             "-fno-sanitize-recover=undefined", "-ffp-contract=off", "-I", HERE, "-I", CSRC, "-w"]
    cmd = ["g++"] + flags
    for s in srcs:
        cmd += ["-x", "c++", s]
    cmd += ["-x", "c++", os.path.join(HERE, "sanitize_driver.cpp"), "-o", out, "-lpthread"]
    subprocess.check_call(cmd)
    return out


if __name__ == "__main__":
    print(build(force=True))

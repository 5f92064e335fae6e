"""The kernel sources under AddressSanitizer and UndefinedBehaviorSanitizer on the CPU (tests/cpu_emu/
sanitize_driver.cpp): an access outside an array in a kernel is a report here instead of a fault on a GPU.
Compiling takes a minute or two and a case a minute or more (the emulation switches contexts at every barrier and
shuffle), so the test runs only when F3M_SANITIZE is set: F3M_SANITIZE=1 runs three cases of ~400 points,
F3M_SANITIZE=<first>,<count>,<points> any others.  F3M_SANITIZE=1 also runs the symmetric near field in 3, 4 and 5 dimensions."""
import os
import subprocess
import sys

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "cpu_emu"))


@pytest.mark.skipif(not os.environ.get("F3M_SANITIZE"), reason="set F3M_SANITIZE=1 to run the kernels under the sanitizers")
def test_kernels_under_address_and_undefined_behaviour_sanitizers():
    import build_emu
    exe = build_emu.build_sanitize_driver()
    spec = os.environ["F3M_SANITIZE"]
    args = spec.split(",") if "," in spec else ["0", "3", "400"]
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0")      # the process ends with the library's caches still held
    r = subprocess.run([exe] + args, env=env, capture_output=True, text=True, timeout=3600)
    print(r.stdout[-4000:])
    print(r.stderr[-4000:])
    assert r.returncode == 0 and "done" in r.stdout
    assert "ERROR: AddressSanitizer" not in r.stderr and "runtime error" not in r.stderr
    if "," in spec:
        return
    # the symmetric near field (one tree, one column, one wavefront per work item) in 3, 4 and 5 dimensions: its LDS block,
    # the skipped boxes of a list, the fixed-point sums
    for shape in (["3", "27", "60", "30"], ["4", "16", "60", "30"], ["5", "32", "60", "30"]):
        env2 = dict(env, F3M_SPLIT_TARGET="1", F3M_NEAR="mfma", F3M_NEAR_FACT="1")
        r = subprocess.run([exe, "0", "1", "500"] + shape, env=env2, capture_output=True, text=True, timeout=3600)
        print(r.stdout[-2000:])
        print(r.stderr[-2000:])
        assert r.returncode == 0 and "done" in r.stdout
        assert "ERROR: AddressSanitizer" not in r.stderr and "runtime error" not in r.stderr

"""visualmesh_amd/csrc/libm_exact.h must return the host C library's bits: the CPU engine's pixel
coordinates come from the host's acosf/sinf/tanf, and on noise images a one-ulp difference in a pixel
coordinate moves a class probability by up to 1e-4. The header compiles for the host too, so it is compared
here with the host libm over EVERY float of the relevant ranges (about 4.5e9 evaluations, a few seconds per
core); the device build of the same source is spot-checked on the GPU in test_gpu_parity.py."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_libm_exact_matches_host_libm_exhaustively(tmp_path):
    exe = str(tmp_path / "libm_exhaustive")
    src = os.path.join(ROOT, "tests", "native", "libm_exhaustive.cpp")
    subprocess.run(["g++", "-O2", "-std=c++17", "-ffp-contract=off", "-mfma", "-pthread",
                    "-I" + os.path.join(ROOT, "visualmesh_amd", "csrc"), src, "-o", exe], check=True)
    threads = str(min(8, os.cpu_count() or 1))
    out = subprocess.run([exe, threads], capture_output=True, text=True, timeout=1500)
    lines = [l.split() for l in out.stdout.strip().splitlines()]
    assert len(lines) == 5, out.stdout + out.stderr
    for name, bad in lines:
        assert int(bad) == 0, "%s: %s results differ from the host C library" % (name, bad)
    assert out.returncode == 0

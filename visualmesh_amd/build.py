"""Build recipes for the native libraries, run on the CPU (hipcc cross-compiles for gfx950).

    python -m visualmesh_amd.build            # build everything that is out of date
    python -m visualmesh_amd.build --force    # rebuild everything

Outputs stay in-tree (visualmesh_amd/lib/*.so) so they travel with the source tree to a GPU machine.
"""
import os
import subprocess
import sys

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
CPP = os.path.join(PKG, "cpp")
LIB = os.path.join(PKG, "lib")
OBJ = os.path.join(PKG, "lib", "obj")
INCLUDE = os.path.join(ROOT, "include")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
CXX = os.environ.get("CXX", "g++")
ARCH = "gfx950"

# Packed-fp32 instructions are switched off for all device code.
HIP_FLAGS = ["--offload-arch=" + ARCH, "-O3", "-std=c++17", "-fPIC", "-I" + INCLUDE, "-I" + CSRC,
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument", "-Wno-inline-asm"]
# Host code that must reproduce the reference's arithmetic: one IEEE operation per step, and sin(x), cos(x) as the two
# C library calls the sources write (merged into sincos() by the compiler, their double results differ in the last bit
# for some arguments).
HOST_EXACT_FLAGS = ["-std=c++14", "-O2", "-ffp-contract=off", "-fno-builtin-sin", "-fno-builtin-cos", "-fPIC", "-Wall", "-Wextra"]

HIP_LIB = os.path.join(LIB, "libvisualmesh_hip.so")
HOST_LIB = os.path.join(LIB, "libvisualmesh_host.so")
HOST_LIB_F64 = os.path.join(LIB, "libvisualmesh_host_f64.so")


def _run(cmd):
    print("+ " + " ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)


def _stale(target, sources):
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(s) > t for s in sources)


def _headers():
    out = [os.path.join(INCLUDE, "visualmesh_hip.h")]
    for d in (CSRC, CPP):
        for base, _, files in os.walk(d):
            out += [os.path.join(base, f) for f in files if f.endswith((".h", ".hpp", ".inc"))]
    return out


def build_hip(force=False):
    """libvisualmesh_hip.so: the HIP kernels and the C ABI of include/visualmesh_hip.h."""
    os.makedirs(OBJ, exist_ok=True)
    headers = _headers()
    objs = []
    units = [
        # project.hip reproduces the reference's operation order: no FMA contraction in that file
        ("project.hip", HIP_FLAGS + ["-ffp-contract=off"]),
        ("conv.hip", HIP_FLAGS),
        ("conv_mfma.hip", HIP_FLAGS),
        ("conv_bf16.hip", HIP_FLAGS),
        ("conv_lds.hip", HIP_FLAGS),
        ("conv_flow.hip", HIP_FLAGS),
        ("conv_narrow.hip", HIP_FLAGS),
        ("detect.hip", HIP_FLAGS),
        ("noalloc.hip", HIP_FLAGS),
        # the double engine: its projection keeps the reference's operation order too
        ("f64.hip", HIP_FLAGS + ["-ffp-contract=off"]),
        ("api.hip", HIP_FLAGS),
    ]
    for name, flags in units:
        src = os.path.join(CSRC, name)
        obj = os.path.join(OBJ, name + ".o")
        if force or _stale(obj, [src] + headers):
            _run([HIPCC] + flags + ["-c", src, "-o", obj])
        objs.append(obj)
    src = os.path.join(CSRC, "host_project.cpp")
    obj = os.path.join(OBJ, "host_project.o")
    if force or _stale(obj, [src] + headers):
        _run([CXX] + HOST_EXACT_FLAGS + ["-c", src, "-o", obj])
    objs.append(obj)
    if force or _stale(HIP_LIB, objs):
        _run([HIPCC, "--offload-arch=" + ARCH, "-shared", "-fPIC", "-o", HIP_LIB] + objs)
    return HIP_LIB


def build_host(force=False):
    """libvisualmesh_host.so: the C++ engine (visualmesh::engine::hip::Engine, Mesh, VisualMesh) behind a
    small C interface so that Python tests and the benchmark drive the real C++ host code."""
    os.makedirs(LIB, exist_ok=True)
    src = os.path.join(PKG, "capi", "host_capi.cpp")
    for target, defines in ((HOST_LIB, []), (HOST_LIB_F64, ["-DVMH_DOUBLE"])):  # Scalar = float, Scalar = double
        if force or _stale(target, [src, HIP_LIB] + _headers()):
            _run([CXX] + HOST_EXACT_FLAGS + defines + ["-I" + CPP, "-I" + INCLUDE, "-shared", src, "-o", target,
                                                       "-L" + LIB, "-lvisualmesh_hip", "-Wl,-rpath,$ORIGIN", "-pthread"])
    return HOST_LIB


def build_all(force=False):
    build_hip(force)
    build_host(force)


if __name__ == "__main__":
    build_all("--force" in sys.argv)

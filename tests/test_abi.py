"""The C ABI library loads without a GPU and exports every symbol include/visualmesh_hip.h declares."""
import ctypes
import os
import re

import pytest

from visualmesh_amd import native

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "visualmesh_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(vmhip_[a-z_0-9]+)\s*\(", text)))


def test_header_and_binding_list_agree():
    assert declared_symbols() == sorted(native.HIP_SYMBOLS)


def test_hip_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(native.HIP_LIB)
    for name in declared_symbols():
        assert hasattr(lib, name), name + " is declared in the header but not exported"


def test_host_library_loads_and_links_the_hip_library():
    lib = native.host()
    for name in ("vmh_mesh_create", "vmh_mesh_lookup", "vmh_visualmesh_create", "vmh_engine_create", "vmh_engine_project",
                 "vmh_engine_classify", "vmh_engine_set_device_lookup", "vmh_engine_stage", "vmh_engine_run", "vmh_engine_fetch", "vmh_engine_result"):
        assert hasattr(lib, name)


def test_struct_layouts_match_the_header():
    # vmhip_lens: 2 int32 + int32 + float + 2 float + 2 float + float = 36 bytes; vmhip_frame holds it by value
    assert ctypes.sizeof(native.Lens) == 36
    assert ctypes.sizeof(native.Layer) == 32
    assert ctypes.sizeof(native.Result) == 40
    assert native.Frame.Rco.offset == 8 and native.Frame.lens.offset == 44 and native.Frame.ranges.offset == 80
    # ranges 80, n_ranges 88 (+4 padding), image 96, fourcc 104 (+4 padding), lookup 112
    assert native.Frame.lookup.offset == 112 and ctypes.sizeof(native.Frame) == 120
    assert ctypes.sizeof(native.LookupExport) == 32 and native.LookupExport.vectors.offset == 8
    # vmhip_detections: four int32, then seven pointers
    assert ctypes.sizeof(native.Detections) == 72
    assert native.Detections.node.offset == 16 and native.Detections.cluster_centre.offset == 64


def test_double_struct_layouts_match_the_header(tmp_path):
    """the _f64 structures as the C compiler lays them out against the ctypes mirrors, and the double host library"""
    import subprocess
    src = tmp_path / "layout.c"
    src.write_text('#include <stdio.h>\n#include <stddef.h>\n#include "visualmesh_hip.h"\nint main(void) { printf("%zu %zu %zu %zu %zu %zu %zu %zu\\n", '
                   'sizeof(vmhip_lens_f64), sizeof(vmhip_layer_f64), sizeof(vmhip_network_f64), sizeof(vmhip_frame_f64), sizeof(vmhip_result_f64), '
                   'offsetof(vmhip_frame_f64, lens), offsetof(vmhip_frame_f64, ranges), offsetof(vmhip_frame_f64, fourcc)); return 0; }\n')
    exe = tmp_path / "layout"
    subprocess.run(["gcc", "-std=c99", "-I" + os.path.join(ROOT, "include"), str(src), "-o", str(exe)], check=True)
    got = [int(v) for v in subprocess.run([str(exe)], stdout=subprocess.PIPE, universal_newlines=True, check=True).stdout.split()]
    want = [ctypes.sizeof(native.Lens64), ctypes.sizeof(native.Layer64), ctypes.sizeof(native.NetworkC64), ctypes.sizeof(native.Frame64),
            ctypes.sizeof(native.Result64), native.Frame64.lens.offset, native.Frame64.ranges.offset, native.Frame64.fourcc.offset]
    assert got == want
    lib = native.host64()
    for name in ("vmh_mesh_create", "vmh_mesh_lookup", "vmh_visualmesh_create", "vmh_engine_create", "vmh_engine_project", "vmh_engine_classify",
                 "vmh_engine_guard_stats"):
        assert hasattr(lib, name)


def build_integration_snippet(directory):
    """the reference's call sites with the engine type changed, compiled as C++14 against the host headers and linked
    with the HIP library; returns the executable"""
    import subprocess
    exe = os.path.join(str(directory), "integration_snippet")
    lib_dir = os.path.dirname(native.HIP_LIB)
    subprocess.run(["g++", "-std=c++14", "-O1", "-Wall", "-Wextra", "-Werror", "-I" + os.path.join(ROOT, "visualmesh_amd", "cpp"),
                    "-I" + os.path.join(ROOT, "include"), os.path.join(ROOT, "tests", "native", "integration_snippet.cpp"),
                    "-L" + lib_dir, "-lvisualmesh_hip", "-Wl,-rpath," + lib_dir, "-o", exe], check=True)
    return exe


def test_reference_call_sites_compile_against_the_host_headers(tmp_path):
    assert os.path.exists(build_integration_snippet(tmp_path))


REFERENCE_CPP = "/root/reference/cpp"


@pytest.mark.skipif(not os.path.isdir(os.path.join(REFERENCE_CPP, "visualmesh")), reason="the reference tree is not mounted here")
def test_engine_header_compiles_against_the_references_own_headers():
    """engine/hip/engine.hpp dropped into the reference tree: its Mesh, VisualMesh, Lens, NetworkStructure, ProjectedMesh and
    ClassifiedMesh are then the reference's (their include directory comes first); syntax and templates only."""
    import subprocess
    cmd = ["g++", "-std=c++14", "-fsyntax-only", "-Wall", "-Wextra", "-I" + REFERENCE_CPP, "-I" + os.path.join(ROOT, "visualmesh_amd", "cpp"),
           "-I" + os.path.join(ROOT, "include"), os.path.join(ROOT, "tests", "native", "reference_interface.cpp")]
    done = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, universal_newlines=True)
    assert done.returncode == 0, done.stdout[-4000:]
    # the reference's headers were really the ones found: a dependency list names them
    deps = subprocess.run(cmd[:2] + ["-MM"] + cmd[3:], stdout=subprocess.PIPE, universal_newlines=True, check=True).stdout
    assert REFERENCE_CPP + "/visualmesh/mesh.hpp" in deps and "visualmesh_amd/cpp/visualmesh/engine/hip/engine.hpp" in deps, deps
    assert "visualmesh_amd/cpp/visualmesh/mesh.hpp" not in deps, deps


@pytest.mark.skipif(not os.path.isdir(os.path.join(REFERENCE_CPP, "visualmesh")), reason="the reference tree is not mounted here")
def test_converting_constructors_match_the_references(tmp_path):
    """Mesh<float>(Mesh<double>), Mesh<double>(Mesh<float>) and VisualMesh<float>(VisualMesh<double>) (reference
    mesh.hpp:476-488, visualmesh.hpp:104-110): one source compiled against the host headers here and against the
    reference's; nodes, neighbours and the lookup ranges of the converted meshes must come out the same, bit for bit."""
    import subprocess
    from visualmesh_amd import build as vm_build
    src = os.path.join(ROOT, "tests", "native", "convert_scalar.cpp")
    printed = []
    for name, include in (("ours", os.path.join(ROOT, "visualmesh_amd", "cpp")), ("reference", REFERENCE_CPP)):
        exe = str(tmp_path / ("convert_" + name))
        flags = [f for f in vm_build.HOST_EXACT_FLAGS if f not in ("-fPIC", "-Wall", "-Wextra")]
        subprocess.run(["g++"] + flags + ["-I" + include, src, "-o", exe], check=True)
        printed.append(subprocess.run([exe], stdout=subprocess.PIPE, universal_newlines=True, check=True).stdout)
    assert printed[0] == printed[1]
    lines = printed[0].splitlines()
    assert len(lines) == 30 and all("ranges 0:" not in line for line in lines if "lens 0" in line), printed[0]
    # a converted mesh keeps the node count of the mesh it came from, not of one generated in its own scalar type
    count = {line.split(" nodes ")[0]: int(line.split(" nodes ")[1].split()[0]) for line in lines if " nodes " in line}
    assert count["double->float"] == count["double"] and count["float->double"] == count["float"]


def test_engine_can_be_compiled_out():
    """VISUALMESH_DISABLE_HIP (what cmake/HipEngine.cmake defines when BUILD_HIP_ENGINE is off, as the reference does for
    its OpenCL and Vulkan engines) leaves an empty header: nothing of the HIP library is needed then."""
    import subprocess
    src = '#include "visualmesh/engine/hip/engine.hpp"\n#ifdef VISUALMESH_HIP_H\n#error the C ABI header was included\n#endif\nint main() { return 0; }\n'
    done = subprocess.run(["g++", "-std=c++14", "-fsyntax-only", "-DVISUALMESH_DISABLE_HIP", "-I" + os.path.join(ROOT, "visualmesh_amd", "cpp"), "-x", "c++", "-"],
                          input=src, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, universal_newlines=True)
    assert done.returncode == 0, done.stdout[-2000:]


def test_bf16_kernels_do_not_spill(tmp_path):
    """conv_bf16.hip places the weights of nearly all instantiations in accumulation registers (an "a" constraint). A
    kernel that spills with its weights placed like that gets wrong results from this compiler: a weight's four
    registers go to scratch as three words plus one word parked in a vector register, and only the three come back
    before the matrix instruction reads all four. So no instantiation may have a scratch segment at all, pinned or not
    (the hand-counted waits of the kernel also assume that the compiler adds no memory traffic of its own): compile the
    file to assembly with the library's flags and check every kernel, and that the weights are where the source says."""
    import subprocess
    from visualmesh_amd import build as vm_build
    out = tmp_path / "conv_bf16.s"
    flags = [f for f in vm_build.HIP_FLAGS if f != "-fPIC"]
    subprocess.run([vm_build.HIPCC] + flags + ["-S", "--cuda-device-only", "-o", str(out), os.path.join(vm_build.CSRC, "conv_bf16.hip")],
                   check=True, stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)
    text = out.read_text()
    checked = 0
    for m in re.finditer(r"\n(_ZN12_GLOBAL__N_119vm_conv_bf16_kernelILi7ELi(\d)ELi(\d)ELi(\d)EEEv\S+?):", text):
        name, rows_in, rows_out, activation = m.group(1), int(m.group(2)), int(m.group(3)), int(m.group(4))
        body = text[m.end():text.index(".Lfunc_end", m.end())]
        from_agprs = sum(1 for line in body.splitlines() if line.strip().startswith("v_mfma") and line.split(",")[1].strip().startswith("a["))
        total = sum(1 for line in body.splitlines() if line.strip().startswith("v_mfma"))
        scratch = int(re.search(r"\.private_segment_fixed_size:\s+(\d+)", text[text.index(".name:           " + name):]).group(1))
        expected_in_agprs = not (rows_in == 0 and rows_out == 2 and activation in (0, 3))
        assert (from_agprs > total // 2) == expected_in_agprs, (name, from_agprs, total)
        assert scratch == 0, name + " spills"
        assert "Folded Reload" not in body and "scratch_" not in body, name
        checked += 1
    assert checked == 36

"""ctypes bindings of the two native libraries.

    hip()    libvisualmesh_hip.so       the C ABI of include/visualmesh_hip.h (kernels + device state)
    host()   libvisualmesh_host.so      the C++ host code (Mesh, VisualMesh, visualmesh::engine::hip::Engine)
                                        behind a small C interface, instantiated for Scalar = float
    host64() libvisualmesh_host_f64.so  the same for Scalar = double (Mesh<double, ...>, Engine<double>)

There is no fallback: if a library has not been built, loading raises, and every call that needs a GPU
fails with the library's own error when none is present.
"""
import ctypes as C
import os

import numpy as np

PKG = os.path.dirname(os.path.abspath(__file__))
HIP_LIB = os.path.join(PKG, "lib", "libvisualmesh_hip.so")
HOST_LIB = os.path.join(PKG, "lib", "libvisualmesh_host.so")
HOST_LIB_F64 = os.path.join(PKG, "lib", "libvisualmesh_host_f64.so")

OK, ERR_HIP, ERR_FORMAT, ERR_LENS, ERR_ARGUMENT, ERR_CAPACITY = 0, -1, -2, -3, -4, -5
FP32, BF16, FP64, SPLIT = 0, 1, 2, 3
DEBUG_FLOW_POLL_LIMIT, DEBUG_PROJECTION_ERROR, DEBUG_EDGE_BAND, DEBUG_WIDE_OFFSETS, DEBUG_STAMP_ROW_BITS = 0, 1, 2, 3, 4

# every symbol include/visualmesh_hip.h declares
HIP_SYMBOLS = [
    "vmhip_last_error", "vmhip_engine_create", "vmhip_engine_destroy", "vmhip_engine_n_classes", "vmhip_mesh_upload",
    "vmhip_mesh_release", "vmhip_project", "vmhip_classify", "vmhip_classify_batch", "vmhip_batch_create",
    "vmhip_batch_destroy", "vmhip_mesh_attach_tree", "vmhip_batch_stage", "vmhip_batch_stage_async", "vmhip_batch_ranges", "vmhip_batch_export", "vmhip_batch_run", "vmhip_batch_run_async", "vmhip_batch_wait", "vmhip_batch_counts", "vmhip_batch_fetch", "vmhip_batch_fetch_async", "vmhip_batch_fetch_wait", "vmhip_batch_fetch_packed_size", "vmhip_batch_fetch_packed_async", "vmhip_batch_detect", "vmhip_host_alloc", "vmhip_host_free",
    "vmhip_batch_profile", "vmhip_batch_profile_read", "vmhip_selftest_libm", "vmhip_selftest_copy", "vmhip_selftest_stream", "vmhip_project_noalloc", "vmhip_debug_set", "vmhip_batch_guard_stats", "vmhip_batch_graph_stats",
    "vmhip_engine_create_f64", "vmhip_engine_destroy_f64", "vmhip_engine_n_classes_f64", "vmhip_mesh_upload_f64", "vmhip_mesh_release_f64",
    "vmhip_project_f64", "vmhip_classify_f64", "vmhip_engine_guard_stats_f64",
]


class VisualMeshError(RuntimeError):
    def __init__(self, code, message):
        super().__init__("%s (status %d)" % (message, code))
        self.code = code


class Lens(C.Structure):
    _fields_ = [("width", C.c_int32), ("height", C.c_int32), ("projection", C.c_int32), ("focal_length", C.c_float),
                ("centre", C.c_float * 2), ("k", C.c_float * 2), ("fov", C.c_float)]


def make_lens(width, height, projection, focal_length, fov, centre=(0.0, 0.0), k=(0.0, 0.0)):
    return Lens(width, height, projection, focal_length, (C.c_float * 2)(*centre), (C.c_float * 2)(*k), fov)


class Layer(C.Structure):
    _fields_ = [("n_in", C.c_int32), ("n_out", C.c_int32), ("activation", C.c_int32), ("weights", C.POINTER(C.c_float)),
                ("biases", C.POINTER(C.c_float))]


class NetworkC(C.Structure):
    _fields_ = [("n_groups", C.c_int32), ("group_sizes", C.POINTER(C.c_int32)), ("layers", C.POINTER(Layer))]


class Frame(C.Structure):
    _fields_ = [("mesh", C.c_void_p), ("Rco", C.c_float * 9), ("lens", Lens), ("ranges", C.POINTER(C.c_int32)),
                ("n_ranges", C.c_int32), ("image", C.c_void_p), ("fourcc", C.c_uint32), ("lookup", C.c_void_p)]


class LookupExport(C.Structure):
    _fields_ = [("capacity", C.c_int32), ("n_points", C.c_int32), ("vectors", C.POINTER(C.c_float)),
                ("graph", C.POINTER(C.c_int32)), ("pixels", C.POINTER(C.c_float))]


class Detections(C.Structure):
    _fields_ = [("capacity", C.c_int32), ("cluster_capacity", C.c_int32), ("n_detections", C.c_int32), ("n_clusters", C.c_int32),
                ("node", C.POINTER(C.c_int32)), ("pixel", C.POINTER(C.c_float)), ("probability", C.POINTER(C.c_float)),
                ("cluster", C.POINTER(C.c_int32)), ("cluster_size", C.POINTER(C.c_int32)), ("cluster_box", C.POINTER(C.c_float)),
                ("cluster_centre", C.POINTER(C.c_float))]


class ProjectionDevice(C.Structure):
    """vmhip_projection_device: where vmhip_project_noalloc writes; every pointer must be addressable by the device"""
    _fields_ = [("capacity", C.c_int32), ("n_visible", C.POINTER(C.c_int32)), ("pixel_coordinates", C.POINTER(C.c_float)),
                ("global_indices", C.POINTER(C.c_int32)), ("neighbourhood", C.POINTER(C.c_int32))]


class Result(C.Structure):
    _fields_ = [("capacity", C.c_int32), ("n_visible", C.c_int32), ("pixel_coordinates", C.POINTER(C.c_float)),
                ("global_indices", C.POINTER(C.c_int32)), ("neighbourhood", C.POINTER(C.c_int32)),
                ("classifications", C.POINTER(C.c_float))]


class Lens64(C.Structure):
    """vmhip_lens_f64"""
    _fields_ = [("width", C.c_int32), ("height", C.c_int32), ("projection", C.c_int32), ("focal_length", C.c_double),
                ("centre", C.c_double * 2), ("k", C.c_double * 2), ("fov", C.c_double)]


def make_lens64(width, height, projection, focal_length, fov, centre=(0.0, 0.0), k=(0.0, 0.0)):
    return Lens64(width, height, projection, focal_length, (C.c_double * 2)(*centre), (C.c_double * 2)(*k), fov)


class Layer64(C.Structure):
    _fields_ = [("n_in", C.c_int32), ("n_out", C.c_int32), ("activation", C.c_int32), ("weights", C.POINTER(C.c_double)),
                ("biases", C.POINTER(C.c_double))]


class NetworkC64(C.Structure):
    _fields_ = [("n_groups", C.c_int32), ("group_sizes", C.POINTER(C.c_int32)), ("layers", C.POINTER(Layer64))]


class Frame64(C.Structure):
    _fields_ = [("mesh", C.c_void_p), ("Rco", C.c_double * 9), ("lens", Lens64), ("ranges", C.POINTER(C.c_int32)),
                ("n_ranges", C.c_int32), ("image", C.c_void_p), ("fourcc", C.c_uint32)]


class Result64(C.Structure):
    _fields_ = [("capacity", C.c_int32), ("n_visible", C.c_int32), ("pixel_coordinates", C.POINTER(C.c_double)),
                ("global_indices", C.POINTER(C.c_int32)), ("neighbourhood", C.POINTER(C.c_int32)),
                ("classifications", C.POINTER(C.c_double))]


def _fp(a):
    return a.ctypes.data_as(C.POINTER(C.c_float))


def _dp(a):
    return a.ctypes.data_as(C.POINTER(C.c_double))


def _ip(a):
    return a.ctypes.data_as(C.POINTER(C.c_int32))


class Network:
    """list of groups, group = list of (weights[n_in, n_out], biases[n_out], activation) -> vmhip_network"""

    def __init__(self, groups):
        self.groups = groups
        self._keep = []
        layers = []
        for g in groups:
            for (w, b, act) in g:
                w = np.ascontiguousarray(w, dtype=np.float32)
                b = np.ascontiguousarray(b, dtype=np.float32)
                self._keep += [w, b]
                layers.append(Layer(w.shape[0], w.shape[1], act, _fp(w), _fp(b)))
        self._layers = (Layer * max(len(layers), 1))(*layers)
        self._sizes = (C.c_int32 * max(len(groups), 1))(*[len(g) for g in groups])
        self.c = NetworkC(len(groups), self._sizes, self._layers)
        self.n_out = groups[-1][-1][0].shape[1] if groups else 4


class Network64:
    """list of groups, group = list of (weights[n_in, n_out], biases[n_out], activation) -> vmhip_network_f64"""

    def __init__(self, groups):
        self.groups = groups
        self._keep = []
        layers = []
        for g in groups:
            for (w, b, act) in g:
                w = np.ascontiguousarray(w, dtype=np.float64)
                b = np.ascontiguousarray(b, dtype=np.float64)
                self._keep += [w, b]
                layers.append(Layer64(w.shape[0], w.shape[1], act, _dp(w), _dp(b)))
        self._layers = (Layer64 * max(len(layers), 1))(*layers)
        self._sizes = (C.c_int32 * max(len(groups), 1))(*[len(g) for g in groups])
        self.c = NetworkC64(len(groups), self._sizes, self._layers)
        self.n_out = groups[-1][-1][0].shape[1] if groups else 4


_hip = None
_host = None
_host64 = None


def hip():
    """libvisualmesh_hip.so with argument types set."""
    global _hip
    if _hip is not None:
        return _hip
    if not os.path.exists(HIP_LIB):
        raise FileNotFoundError(HIP_LIB + " is not built: run `python -m visualmesh_amd.build`")
    L = C.CDLL(HIP_LIB, mode=C.RTLD_GLOBAL)
    vp = C.c_void_p
    L.vmhip_last_error.restype = C.c_char_p
    L.vmhip_engine_create.argtypes = [C.POINTER(NetworkC), C.c_int32, C.c_int32, C.POINTER(vp)]
    L.vmhip_engine_destroy.argtypes = [vp]
    L.vmhip_engine_destroy.restype = None
    L.vmhip_engine_n_classes.argtypes = [vp]
    L.vmhip_mesh_upload.argtypes = [C.POINTER(C.c_float), C.POINTER(C.c_int32), C.c_int32, C.c_int32, C.POINTER(vp)]
    L.vmhip_mesh_release.argtypes = [vp]
    L.vmhip_mesh_release.restype = None
    L.vmhip_project.argtypes = [vp, C.POINTER(Frame), C.POINTER(Result)]
    L.vmhip_classify.argtypes = [vp, C.POINTER(Frame), C.POINTER(Result)]
    L.vmhip_classify_batch.argtypes = [vp, C.POINTER(Frame), C.c_int32, C.POINTER(Result)]
    L.vmhip_batch_create.argtypes = [vp, C.POINTER(vp)]
    L.vmhip_batch_destroy.argtypes = [vp]
    L.vmhip_batch_destroy.restype = None
    L.vmhip_batch_stage.argtypes = [vp, C.POINTER(Frame), C.c_int32, C.c_int32]
    L.vmhip_batch_stage_async.argtypes = [vp, C.POINTER(Frame), C.c_int32, C.c_int32]
    L.vmhip_batch_run.argtypes = [vp]
    L.vmhip_batch_counts.argtypes = [vp, C.POINTER(C.c_int32)]
    L.vmhip_batch_fetch.argtypes = [vp, C.POINTER(Result)]
    L.vmhip_batch_fetch_async.argtypes = [vp, C.POINTER(Result)]
    L.vmhip_batch_fetch_wait.argtypes = [vp]
    L.vmhip_batch_fetch_packed_size.argtypes = [vp]
    L.vmhip_batch_fetch_packed_size.restype = C.c_size_t
    L.vmhip_batch_fetch_packed_async.argtypes = [vp, vp, C.c_size_t, C.POINTER(Result)]
    L.vmhip_batch_run_async.argtypes = [vp]
    L.vmhip_batch_export.argtypes = [vp, C.c_int32, C.POINTER(LookupExport)]
    L.vmhip_batch_ranges.argtypes = [vp, C.c_int32, C.POINTER(C.c_int32), C.c_int32]
    L.vmhip_mesh_attach_tree.argtypes = [vp, vp, C.c_int32]
    L.vmhip_batch_wait.argtypes = [vp]
    L.vmhip_batch_detect.argtypes = [vp, C.c_int32, C.c_float, C.c_int32, C.c_int32, C.POINTER(Detections)]
    L.vmhip_host_alloc.restype = vp
    L.vmhip_host_alloc.argtypes = [C.c_size_t]
    L.vmhip_host_free.restype = None
    L.vmhip_host_free.argtypes = [vp]
    L.vmhip_batch_profile.argtypes = [vp, C.c_int32]
    L.vmhip_batch_profile_read.argtypes = [vp, C.c_int32, C.POINTER(C.c_int32), C.POINTER(C.c_char_p), C.POINTER(C.c_float),
                                           C.POINTER(C.c_int64)]
    L.vmhip_selftest_libm.argtypes = [C.c_int32, C.POINTER(C.c_float), C.POINTER(C.c_float), C.c_int32]
    L.vmhip_selftest_copy.argtypes = [C.c_int64, C.c_int32, C.POINTER(C.c_float)]
    L.vmhip_selftest_stream.argtypes = [C.c_int64, C.c_int32, C.c_int32, C.c_int32, C.POINTER(C.c_float)]
    L.vmhip_debug_set.argtypes = [C.c_int32, C.c_double]
    L.vmhip_batch_guard_stats.argtypes = [vp, C.POINTER(C.c_int64), C.POINTER(C.c_int64), C.POINTER(C.c_int64), C.POINTER(C.c_int64)]
    L.vmhip_batch_graph_stats.argtypes = [vp, C.POINTER(C.c_int64), C.POINTER(C.c_int64), C.POINTER(C.c_int64)]
    L.vmhip_project_noalloc.argtypes = [vp, C.POINTER(C.c_float), C.POINTER(Lens), C.POINTER(C.c_int32), C.c_int32, C.c_int32,
                                        C.POINTER(ProjectionDevice), vp]
    dp = C.POINTER(C.c_double)
    L.vmhip_engine_create_f64.argtypes = [C.POINTER(NetworkC64), C.c_int32, C.POINTER(vp)]
    L.vmhip_engine_destroy_f64.argtypes = [vp]
    L.vmhip_engine_destroy_f64.restype = None
    L.vmhip_engine_n_classes_f64.argtypes = [vp]
    L.vmhip_mesh_upload_f64.argtypes = [dp, C.POINTER(C.c_int32), C.c_int32, C.c_int32, C.POINTER(vp)]
    L.vmhip_mesh_release_f64.argtypes = [vp]
    L.vmhip_mesh_release_f64.restype = None
    L.vmhip_project_f64.argtypes = [vp, C.POINTER(Frame64), C.POINTER(Result64)]
    L.vmhip_classify_f64.argtypes = [vp, C.POINTER(Frame64), C.POINTER(Result64)]
    L.vmhip_engine_guard_stats_f64.argtypes = [vp, C.POINTER(C.c_int64), C.POINTER(C.c_int64)]
    _hip = L
    return L


def hip_check(rc):
    if rc < 0:
        raise VisualMeshError(rc, hip().vmhip_last_error().decode())
    return rc


def guard_stats(batch_ptr):
    """dict(listed, most_listed, overruled, reruns): what the edge guard did in the runs of a vmhip_batch since it was staged"""
    v = [C.c_int64(0) for _ in range(4)]
    hip_check(hip().vmhip_batch_guard_stats(batch_ptr, *[C.byref(x) for x in v]))
    return dict(listed=v[0].value, most_listed=v[1].value, overruled=v[2].value, reruns=v[3].value)


def graph_stats(batch_ptr):
    """dict(captures, graph_launches, eager_launches): how the passes of a vmhip_batch were put on the stream since it was made"""
    v = [C.c_int64(0) for _ in range(3)]
    hip_check(hip().vmhip_batch_graph_stats(batch_ptr, *[C.byref(x) for x in v]))
    return dict(captures=v[0].value, graph_launches=v[1].value, eager_launches=v[2].value)


def copy_probe(nbytes=1 << 30, repeats=5):
    """average milliseconds of a plain device copy kernel of nbytes (read nbytes + write nbytes)"""
    ms = C.c_float(0.0)
    hip_check(hip().vmhip_selftest_copy(nbytes, repeats, C.byref(ms)))
    return float(ms.value)


def stream_probe(rows, read_bytes_per_row, write_bytes_per_row, repeats=20):
    """average milliseconds of a kernel that only reads and writes a layer's bytes (rows: rounded up to 64)"""
    ms = C.c_float(0.0)
    hip_check(hip().vmhip_selftest_stream((int(rows) + 63) // 64 * 64, read_bytes_per_row, write_bytes_per_row, repeats, C.byref(ms)))
    return float(ms.value)


def profile_read(batch_ptr, max_slots=256):
    """[(kernel name, milliseconds, units)] of the last profiled run of a vmhip_batch."""
    L = hip()
    n = C.c_int32(0)
    names = (C.c_char_p * max_slots)()
    ms = (C.c_float * max_slots)()
    units = (C.c_int64 * max_slots)()
    hip_check(L.vmhip_batch_profile_read(batch_ptr, max_slots, C.byref(n), names, ms, units))
    return [(names[i].decode(), float(ms[i]), int(units[i])) for i in range(n.value)]


def host():
    """libvisualmesh_host.so with argument types set."""
    global _host
    if _host is not None:
        return _host
    hip()  # the host library links against it; load it first so a missing build fails with a clear message
    if not os.path.exists(HOST_LIB):
        raise FileNotFoundError(HOST_LIB + " is not built: run `python -m visualmesh_amd.build`")
    L = C.CDLL(HOST_LIB)
    vp = C.c_void_p
    L.vmh_last_error.restype = C.c_char_p
    L.vmh_mesh_create.restype = vp
    L.vmh_mesh_create.argtypes = [C.c_int, C.c_int, C.c_float, C.c_float, C.c_float, C.c_float]
    L.vmh_mesh_destroy.argtypes = [vp]
    L.vmh_mesh_destroy.restype = None
    L.vmh_mesh_n_nodes.argtypes = [vp]
    L.vmh_mesh_n_neighbours.argtypes = [vp]
    L.vmh_mesh_h.argtypes = [vp]
    L.vmh_mesh_h.restype = C.c_float
    L.vmh_mesh_copy.argtypes = [vp, C.POINTER(C.c_float), C.POINTER(C.c_int32)]
    L.vmh_mesh_copy.restype = None
    L.vmh_mesh_lookup.argtypes = [vp, C.POINTER(C.c_float), C.POINTER(Lens), C.POINTER(C.c_int32), C.c_int]
    L.vmh_visualmesh_create.restype = vp
    L.vmh_visualmesh_create.argtypes = [C.c_int, C.c_int] + [C.c_float] * 6
    L.vmh_visualmesh_destroy.argtypes = [vp]
    L.vmh_visualmesh_destroy.restype = None
    L.vmh_visualmesh_n_meshes.argtypes = [vp]
    L.vmh_visualmesh_mesh.restype = vp
    L.vmh_visualmesh_mesh.argtypes = [vp, C.c_int]
    L.vmh_visualmesh_height.restype = vp
    L.vmh_visualmesh_height.argtypes = [vp, C.c_float]
    L.vmh_engine_create.argtypes = [C.POINTER(NetworkC), C.c_int, C.c_int, C.POINTER(vp)]
    L.vmh_engine_destroy.argtypes = [vp]
    L.vmh_engine_destroy.restype = None
    L.vmh_engine_project.argtypes = [vp, vp, C.POINTER(C.c_float), C.POINTER(Lens), C.c_int, C.POINTER(C.c_float),
                                     C.POINTER(C.c_int32), C.POINTER(C.c_int32)]
    L.vmh_engine_classify.argtypes = [vp, vp, C.POINTER(C.c_float), C.POINTER(Lens), vp, C.c_uint32, C.c_int,
                                      C.POINTER(C.c_float), C.POINTER(C.c_int32), C.POINTER(C.c_int32), C.POINTER(C.c_float)]
    L.vmh_engine_time_calls.argtypes = [vp, vp, C.POINTER(C.c_float), C.POINTER(Lens), vp, C.c_uint32, C.c_int, C.POINTER(C.c_double)]
    L.vmh_engine_stage.argtypes = [vp, C.c_int, C.POINTER(vp), C.POINTER(C.c_float), C.POINTER(Lens), C.POINTER(vp),
                                   C.POINTER(C.c_uint32), C.c_int]
    L.vmh_engine_run.argtypes = [vp]
    L.vmh_engine_counts.argtypes = [vp, C.POINTER(C.c_int32), C.c_int]
    L.vmh_engine_fetch.argtypes = [vp]
    L.vmh_engine_result.argtypes = [vp, C.c_int, C.c_int, C.POINTER(C.c_float), C.POINTER(C.c_int32), C.POINTER(C.c_int32),
                                    C.POINTER(C.c_float)]
    L.vmh_engine_lookup_graph.argtypes = [vp, C.c_int, C.c_int, C.c_int, C.POINTER(C.c_float), C.POINTER(C.c_int32), C.POINTER(C.c_float)]
    L.vmh_engine_native_batch.restype = vp
    L.vmh_engine_native_batch.argtypes = [vp]
    L.vmh_engine_clear_cache.argtypes = [vp]
    L.vmh_engine_clear_cache.restype = None
    L.vmh_engine_set_cache_limit.argtypes = [vp, C.c_uint64]
    L.vmh_engine_set_cache_limit.restype = None
    L.vmh_engine_set_device_lookup.argtypes = [vp, C.c_int]
    L.vmh_engine_set_device_lookup.restype = None
    L.vmh_engine_cache_info.argtypes = [vp, C.POINTER(C.c_uint64)]
    L.vmh_model_load.restype = vp
    L.vmh_model_load.argtypes = [C.c_char_p]
    L.vmh_model_free.argtypes = [vp]
    L.vmh_model_free.restype = None
    L.vmh_model_info.argtypes = [vp, C.c_char_p, C.c_char_p, C.c_int, C.POINTER(C.c_float), C.POINTER(C.c_float)]
    L.vmh_model_group_size.argtypes = [vp, C.c_int]
    L.vmh_model_layer.argtypes = [vp, C.c_int, C.c_int, C.POINTER(C.c_int), C.POINTER(C.c_int), C.POINTER(C.c_int),
                                  C.POINTER(C.c_float), C.POINTER(C.c_float)]
    L.vmh_lens_load.argtypes = [C.c_char_p, C.c_int, C.c_int, C.POINTER(Lens), C.POINTER(C.c_float)]
    fpp, ipp = C.POINTER(C.POINTER(C.c_float)), C.POINTER(C.POINTER(C.c_int32))
    L.vmh_pipeline_create.argtypes = [C.POINTER(NetworkC), C.c_int, C.c_int, C.POINTER(vp)]
    L.vmh_pipeline_destroy.argtypes = [vp]
    L.vmh_pipeline_destroy.restype = None
    L.vmh_pipeline_submit.argtypes = [vp, C.c_int, C.POINTER(vp), C.POINTER(C.c_float), C.POINTER(Lens), C.POINTER(vp), C.POINTER(C.c_uint32)]
    L.vmh_pipeline_result.argtypes = [vp, C.c_int, fpp, ipp, ipp, fpp]
    L.vmh_pipeline_n_classes.argtypes = [vp]
    L.vmh_pipeline_graph_stats.argtypes = [vp, C.POINTER(C.c_int64), C.POINTER(C.c_int64), C.POINTER(C.c_int64)]
    _host = L
    return L


def host64():
    """libvisualmesh_host_f64.so (Scalar = double) with argument types set."""
    global _host64
    if _host64 is not None:
        return _host64
    hip()
    if not os.path.exists(HOST_LIB_F64):
        raise FileNotFoundError(HOST_LIB_F64 + " is not built: run `python -m visualmesh_amd.build`")
    L = C.CDLL(HOST_LIB_F64)
    vp, dp, ip = C.c_void_p, C.POINTER(C.c_double), C.POINTER(C.c_int32)
    L.vmh_last_error.restype = C.c_char_p
    L.vmh_mesh_create.restype = vp
    L.vmh_mesh_create.argtypes = [C.c_int, C.c_int, C.c_double, C.c_double, C.c_double, C.c_double]
    L.vmh_mesh_destroy.argtypes = [vp]
    L.vmh_mesh_destroy.restype = None
    L.vmh_mesh_n_nodes.argtypes = [vp]
    L.vmh_mesh_n_neighbours.argtypes = [vp]
    L.vmh_mesh_h.argtypes = [vp]
    L.vmh_mesh_h.restype = C.c_double
    L.vmh_mesh_copy.argtypes = [vp, dp, ip]
    L.vmh_mesh_copy.restype = None
    L.vmh_mesh_lookup.argtypes = [vp, dp, C.POINTER(Lens64), ip, C.c_int]
    L.vmh_visualmesh_create.restype = vp
    L.vmh_visualmesh_create.argtypes = [C.c_int, C.c_int] + [C.c_double] * 6
    L.vmh_visualmesh_destroy.argtypes = [vp]
    L.vmh_visualmesh_destroy.restype = None
    L.vmh_visualmesh_n_meshes.argtypes = [vp]
    L.vmh_visualmesh_mesh.restype = vp
    L.vmh_visualmesh_mesh.argtypes = [vp, C.c_int]
    L.vmh_visualmesh_height.restype = vp
    L.vmh_visualmesh_height.argtypes = [vp, C.c_double]
    L.vmh_engine_create.argtypes = [C.POINTER(NetworkC64), C.c_int, C.c_int, C.POINTER(vp)]
    L.vmh_engine_destroy.argtypes = [vp]
    L.vmh_engine_destroy.restype = None
    L.vmh_engine_project.argtypes = [vp, vp, dp, C.POINTER(Lens64), C.c_int, dp, ip, ip]
    L.vmh_engine_classify.argtypes = [vp, vp, dp, C.POINTER(Lens64), vp, C.c_uint32, C.c_int, dp, ip, ip, dp]
    L.vmh_engine_guard_stats.argtypes = [vp, C.POINTER(C.c_int64), C.POINTER(C.c_int64)]
    _host64 = L
    return L


def host_check(rc, lib=None):
    if rc < 0:
        msg = (lib or host()).vmh_last_error().decode()
        if rc == ERR_FORMAT:
            raise ValueError(msg)
        raise VisualMeshError(rc, msg)
    return rc


class _Pinned:
    """owner of one page-locked allocation; freed when the last array viewing it goes away"""

    def __init__(self, nbytes):
        self.ptr = hip().vmhip_host_alloc(nbytes)
        if not self.ptr:
            raise MemoryError("vmhip_host_alloc(%d) failed" % nbytes)
        self.buffer = (C.c_uint8 * max(nbytes, 1)).from_address(self.ptr)
        self.buffer._owner = self  # numpy keeps the ctypes buffer alive; the buffer keeps this object alive

    def __del__(self):
        if getattr(self, "ptr", None):
            hip().vmhip_host_free(self.ptr)
            self.ptr = None


def pinned_empty(shape, dtype=np.uint8):
    """numpy array in page-locked host memory (vmhip_host_alloc): the place for camera images that go to the device"""
    dtype = np.dtype(dtype)
    n = int(np.prod(shape)) * dtype.itemsize
    owner = _Pinned(n)
    return np.frombuffer(owner.buffer, dtype=np.uint8, count=n).view(dtype).reshape(shape)

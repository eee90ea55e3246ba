"""vmhip_project_noalloc (kernel launches only, workspace inside the library) against vmhip_project, through the C ABI:
two calls in a row on one device, the second on a smaller input, every output bit for bit."""
import ctypes as C
import math

import numpy as np
import pytest

from visualmesh_amd import engine as eng
from visualmesh_amd import native
from visualmesh_amd import workloads as wl

pytestmark = pytest.mark.gpu


ProjectionDevice = native.ProjectionDevice


def _fp(a):
    return a.ctypes.data_as(C.POINTER(C.c_float))


def _ip(a):
    return a.ctypes.data_as(C.POINTER(C.c_int32))


def _device_wait():
    hip_runtime = C.CDLL("libamdhip64.so")
    assert hip_runtime.hipDeviceSynchronize() == 0


def _both_ways(L, engine, mesh_handle, mesh, Hoc, lens):
    """(vmhip_project's outputs, vmhip_project_noalloc's outputs) for one pose"""
    nn = mesh.n_neighbours
    H = np.ascontiguousarray(Hoc, dtype=np.float32)
    ranges = np.ascontiguousarray(mesh.lookup(H, lens), dtype=np.int32)
    n_cand = int((ranges[:, 1] - ranges[:, 0]).sum())
    Rco = np.ascontiguousarray(H[:3, :3].T)

    # the existing entry point: host arrays
    px = np.zeros((n_cand, 2), np.float32)
    gidx = np.zeros(n_cand, np.int32)
    nb = np.zeros((n_cand + 1, nn), np.int32)
    frame = native.Frame(mesh_handle, (C.c_float * 9)(*Rco.ravel()), lens, _ip(ranges), len(ranges), None, 0, None)
    result = native.Result(n_cand, 0, _fp(px), _ip(gidx), _ip(nb), None)
    native.hip_check(L.vmhip_project(engine, C.byref(frame), C.byref(result)))
    V = result.n_visible
    want = dict(V=V, px=px[:V].copy(), gidx=gidx[:V].copy(), nb=nb[:V + 1].copy())

    # the entry point that allocates nothing: everything the device touches is page-locked memory it can address
    d_ranges = native.pinned_empty(ranges.shape, np.int32)
    d_ranges[...] = ranges
    d_V = native.pinned_empty((1,), np.int32)
    d_px = native.pinned_empty((n_cand, 2), np.float32)
    d_gidx = native.pinned_empty((n_cand,), np.int32)
    d_nb = native.pinned_empty((n_cand + 1, nn), np.int32)
    d_V[0] = -7
    d_px[...] = np.nan
    d_gidx[...] = -1
    d_nb[...] = -1
    out = ProjectionDevice(n_cand, _ip(d_V), _fp(d_px), _ip(d_gidx), _ip(d_nb))
    native.hip_check(L.vmhip_project_noalloc(mesh_handle, _fp(Rco), C.byref(lens), _ip(d_ranges), len(ranges), n_cand, C.byref(out), None))
    _device_wait()
    V2 = int(d_V[0])
    got = dict(V=V2, px=d_px[:max(V2, 0)].copy(), gidx=d_gidx[:max(V2, 0)].copy(), nb=d_nb[:max(V2, 0) + 1].copy())
    return want, got, (ranges, n_cand)


def _assert_same(want, got, label):
    assert got["V"] == want["V"], "%s: visible count %d != %d" % (label, got["V"], want["V"])
    assert np.array_equal(got["gidx"], want["gidx"]), label + ": global indices differ"
    assert np.array_equal(got["nb"], want["nb"]), label + ": neighbourhood differs"
    assert np.array_equal(got["px"].view(np.uint32), want["px"].view(np.uint32)), label + ": pixel bits differ"


def test_projection_without_allocation_matches_vmhip_project():
    L = native.hip()
    empty = native.Network([])
    engine = C.c_void_p()
    native.hip_check(L.vmhip_engine_create(C.byref(empty.c), 6, native.FP32, C.byref(engine)))

    big = eng.Mesh(wl.RING6, wl.SPHERE, 0.0949, 1.2, 6.0, 20.0)      # configuration 1's mesh, 121 083 nodes
    small = eng.Mesh(wl.RING6, wl.SPHERE, 0.0949, 1.0, 3.0, 8.0)
    handles = []
    for m in (big, small):
        rays, nbr = m.arrays()
        h = C.c_void_p()
        native.hip_check(L.vmhip_mesh_upload(_fp(rays), _ip(nbr), m.n_nodes, m.n_neighbours, C.byref(h)))
        handles.append(h)

    lens_big = native.make_lens(1280, 1024, wl.EQUISOLID, 420.0, math.pi)
    lens_small = native.make_lens(320, 256, wl.RECTILINEAR, 180.0, math.pi / 2)
    Hoc_big = wl.make_hoc(1.2, math.radians(30.0), math.radians(3.0), math.radians(-2.0))
    Hoc_small = wl.make_hoc(1.0, math.radians(50.0), math.radians(-4.0), math.radians(1.0))

    # first call: configuration 1's geometry; second call right after it: a smaller mesh, lens and view
    want, got, _ = _both_ways(L, engine, handles[0], big, Hoc_big, lens_big)
    print("first call: V =", want["V"], flush=True)
    assert want["V"] > 50000
    _assert_same(want, got, "first call")
    want, got, (ranges, n_cand) = _both_ways(L, engine, handles[1], small, Hoc_small, lens_small)
    print("second call: V =", want["V"], flush=True)
    assert 100 < want["V"] < 50000
    _assert_same(want, got, "second call (smaller)")
    # and the first input once more: what the smaller call left in the workspace does not show
    want, got, _ = _both_ways(L, engine, handles[0], big, Hoc_big, lens_big)
    _assert_same(want, got, "third call")

    # The reverse lookup carries an 8-bit run stamp: after 255 calls the count starts again and the table is cleared on the
    # device. The big mesh's entries, stamped by the call above, must not look current again to any later call.
    for call in range(300):
        want, got, (ranges, n_cand) = _both_ways(L, engine, handles[1], small, Hoc_small, lens_small)
        _assert_same(want, got, "call %d on the smaller input" % call)

    # a range table that does not sum to the stated candidate count is rejected on the device, nothing else is written
    d_ranges = native.pinned_empty(ranges.shape, np.int32)
    d_ranges[...] = ranges
    d_V = native.pinned_empty((1,), np.int32)
    d_px = native.pinned_empty((n_cand + 256, 2), np.float32)
    d_gidx = native.pinned_empty((n_cand + 256,), np.int32)
    d_nb = native.pinned_empty((n_cand + 257, 6), np.int32)
    d_V[0] = 5
    d_gidx[...] = -1
    out = ProjectionDevice(n_cand + 256, _ip(d_V), _fp(d_px), _ip(d_gidx), _ip(d_nb))
    Rco = np.ascontiguousarray(np.asarray(Hoc_small, np.float32)[:3, :3].T)
    native.hip_check(L.vmhip_project_noalloc(handles[1], _fp(Rco), C.byref(lens_small), _ip(d_ranges), len(ranges), n_cand + 3, C.byref(out), None))
    _device_wait()
    assert int(d_V[0]) == -1 and (d_gidx == -1).all()

    # sizes beyond the workspace are refused with the limit named, before anything is launched
    out = ProjectionDevice(600000, _ip(d_V), _fp(d_px), _ip(d_gidx), _ip(d_nb))
    rc = L.vmhip_project_noalloc(handles[1], _fp(Rco), C.byref(lens_small), _ip(d_ranges), len(ranges), 600000, C.byref(out), None)
    assert rc == native.ERR_CAPACITY and b"VMHIP_NOALLOC_MAX_CANDIDATES" in L.vmhip_last_error()
    rc = L.vmhip_project_noalloc(handles[1], _fp(Rco), C.byref(lens_small), _ip(d_ranges), 70000, n_cand, C.byref(out), None)
    assert rc == native.ERR_CAPACITY and b"VMHIP_NOALLOC_MAX_RANGES" in L.vmhip_last_error()

    for h in handles:
        L.vmhip_mesh_release(h)
    L.vmhip_engine_destroy(engine)


def test_projection_without_allocation_inside_a_captured_graph():
    """The use the entry point names first: one call captured into a HIP graph on a stream of the caller's, replayed
    past the point where the 8-bit run stamp starts again (255 calls), with eager calls on another input and waits
    between the replays. Every replay checked leaves vmhip_project's outputs; a frame without candidates leaves a
    visible count of zero and its null row."""
    hip_runtime = C.CDLL("libamdhip64.so")
    for fn in ("hipStreamCreate", "hipStreamBeginCapture", "hipStreamEndCapture", "hipGraphInstantiate", "hipGraphLaunch", "hipStreamSynchronize",
               "hipGraphExecDestroy", "hipGraphDestroy", "hipStreamDestroy"):
        getattr(hip_runtime, fn).restype = C.c_int
    hip_runtime.hipStreamBeginCapture.argtypes = [C.c_void_p, C.c_int]
    hip_runtime.hipStreamEndCapture.argtypes = [C.c_void_p, C.POINTER(C.c_void_p)]
    hip_runtime.hipGraphInstantiate.argtypes = [C.POINTER(C.c_void_p), C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t]
    hip_runtime.hipGraphLaunch.argtypes = [C.c_void_p, C.c_void_p]
    hip_runtime.hipStreamSynchronize.argtypes = [C.c_void_p]
    hip_runtime.hipGraphExecDestroy.argtypes = [C.c_void_p]
    hip_runtime.hipGraphDestroy.argtypes = [C.c_void_p]
    hip_runtime.hipStreamDestroy.argtypes = [C.c_void_p]

    L = native.hip()
    empty = native.Network([])
    engine = C.c_void_p()
    native.hip_check(L.vmhip_engine_create(C.byref(empty.c), 6, native.FP32, C.byref(engine)))
    mesh = eng.Mesh(wl.RING6, wl.SPHERE, 0.0949, 1.0, 3.0, 8.0)
    other = eng.Mesh(wl.RING6, wl.SPHERE, 0.0949, 1.2, 4.0, 10.0)
    handles = []
    for m in (mesh, other):
        rays, nbr = m.arrays()
        h = C.c_void_p()
        native.hip_check(L.vmhip_mesh_upload(_fp(rays), _ip(nbr), m.n_nodes, m.n_neighbours, C.byref(h)))
        handles.append(h)
    lens = native.make_lens(320, 256, wl.RECTILINEAR, 180.0, math.pi / 2)
    Hoc = wl.make_hoc(1.0, math.radians(50.0), math.radians(-4.0), math.radians(1.0))
    Hoc_other = wl.make_hoc(1.2, math.radians(35.0), math.radians(2.0), math.radians(-3.0))
    want, got, (ranges, n_cand) = _both_ways(L, engine, handles[0], mesh, Hoc, lens)
    _assert_same(want, got, "eager call")
    V = want["V"]
    assert V > 100

    nn = mesh.n_neighbours
    d_ranges = native.pinned_empty(ranges.shape, np.int32)
    d_ranges[...] = ranges
    d_V = native.pinned_empty((1,), np.int32)
    d_px = native.pinned_empty((n_cand, 2), np.float32)
    d_gidx = native.pinned_empty((n_cand,), np.int32)
    d_nb = native.pinned_empty((n_cand + 1, nn), np.int32)
    out = ProjectionDevice(n_cand, _ip(d_V), _fp(d_px), _ip(d_gidx), _ip(d_nb))
    Rco = np.ascontiguousarray(np.asarray(Hoc, np.float32)[:3, :3].T)

    stream, graph, graph_exec = C.c_void_p(), C.c_void_p(), C.c_void_p()
    assert hip_runtime.hipStreamCreate(C.byref(stream)) == 0
    assert hip_runtime.hipStreamBeginCapture(stream, 1) == 0  # hipStreamCaptureModeThreadLocal
    rc = L.vmhip_project_noalloc(handles[0], _fp(Rco), C.byref(lens), _ip(d_ranges), len(ranges), n_cand, C.byref(out), stream)
    assert hip_runtime.hipStreamEndCapture(stream, C.byref(graph)) == 0
    native.hip_check(rc)
    assert hip_runtime.hipGraphInstantiate(C.byref(graph_exec), graph, None, None, 0) == 0
    for replay in range(300):
        checked = replay < 4 or replay % 50 == 0 or 250 <= replay < 262 or replay == 299
        if checked:
            d_V[0] = -7
            d_px[...] = np.nan
            d_gidx[...] = -1
            d_nb[...] = -1
        assert hip_runtime.hipGraphLaunch(graph_exec, stream) == 0
        assert hip_runtime.hipStreamSynchronize(stream) == 0
        if checked:
            got = dict(V=int(d_V[0]), px=d_px[:V].copy(), gidx=d_gidx[:V].copy(), nb=d_nb[:V + 1].copy())
            _assert_same(want, got, "replay %d" % replay)
            # an eager call on another mesh and view between the replays: it shares the workspace, not the outputs
            w2, g2, _ = _both_ways(L, engine, handles[1], other, Hoc_other, lens)
            _assert_same(w2, g2, "eager call after replay %d" % replay)
    assert hip_runtime.hipGraphExecDestroy(graph_exec) == 0 and hip_runtime.hipGraphDestroy(graph) == 0 and hip_runtime.hipStreamDestroy(stream) == 0

    # no candidates at all: a visible count of zero and the null row, nothing else
    d_V[0] = -7
    d_nb[...] = -1
    native.hip_check(L.vmhip_project_noalloc(handles[0], _fp(Rco), C.byref(lens), _ip(d_ranges), 0, 0, C.byref(out), None))
    _device_wait()
    assert int(d_V[0]) == 0 and (d_nb[0] == 0).all() and (d_nb[1:] == -1).all()

    for h in handles:
        L.vmhip_mesh_release(h)
    L.vmhip_engine_destroy(engine)

"""Python face of the C++ host code: Mesh, VisualMesh and the HIP Engine.

These classes only marshal numpy arrays in and out of libvisualmesh_host.so; mesh generation, the BSP
lookup and the engine logic are the C++ in visualmesh_amd/cpp, the device work is libvisualmesh_hip.so.
The call shapes mirror the reference's engine interface: engine(mesh, Hoc, lens) projects,
engine(mesh, Hoc, lens, image, fourcc) classifies, `mesh` may be a Mesh or a VisualMesh.
"""
import ctypes as C

import numpy as np

from . import native
from .native import Lens, Network, make_lens  # noqa: F401  (re-exported)


def _fp(a):
    return a.ctypes.data_as(C.POINTER(C.c_float))


def _ip(a):
    return a.ctypes.data_as(C.POINTER(C.c_int32))


class Mesh:
    def __init__(self, model=None, shape=None, radius=None, h=None, k=None, max_distance=None, _ptr=None, _owner=None):
        self._lib = native.host()
        if _ptr is None:
            _ptr = self._lib.vmh_mesh_create(model, shape, radius, h, k, max_distance)
            if not _ptr:
                raise RuntimeError("mesh construction failed: " + self._lib.vmh_last_error().decode())
            self._owned = True
        else:
            self._owned = False
        self._owner = _owner  # keeps a VisualMesh alive while one of its meshes is in use
        self.ptr = _ptr
        self.n_nodes = self._lib.vmh_mesh_n_nodes(_ptr)
        self.n_neighbours = self._lib.vmh_mesh_n_neighbours(_ptr)
        self.h = self._lib.vmh_mesh_h(_ptr)
        self._arrays = None

    def __del__(self):
        if getattr(self, "_owned", False) and self.ptr:
            self._lib.vmh_mesh_destroy(self.ptr)
            self.ptr = None

    def arrays(self):
        """(rays[n,3] float32, neighbours[n,nn] int32) in mesh order"""
        if self._arrays is None:
            rays = np.zeros((self.n_nodes, 3), np.float32)
            nbr = np.zeros((self.n_nodes, self.n_neighbours), np.int32)
            self._lib.vmh_mesh_copy(self.ptr, _fp(rays), _ip(nbr))
            self._arrays = (rays, nbr)
        return self._arrays

    def lookup(self, Hoc, lens):
        H = np.ascontiguousarray(Hoc, dtype=np.float32)
        cap = 4096
        while True:
            r = np.zeros((cap, 2), np.int32)
            n = native.host_check(self._lib.vmh_mesh_lookup(self.ptr, _fp(H), C.byref(lens), _ip(r), cap))
            if n <= cap:
                return r[:n].copy()
            cap = n

    def height(self, h):
        return self


class VisualMesh:
    def __init__(self, model, shape, radius, min_h, max_h, k, max_error, max_distance):
        self._lib = native.host()
        self.ptr = self._lib.vmh_visualmesh_create(model, shape, radius, min_h, max_h, k, max_error, max_distance)
        if not self.ptr:
            raise RuntimeError("visual mesh construction failed: " + self._lib.vmh_last_error().decode())
        n = self._lib.vmh_visualmesh_n_meshes(self.ptr)
        self.meshes = [Mesh(_ptr=self._lib.vmh_visualmesh_mesh(self.ptr, i), _owner=None) for i in range(n)]
        self._by_ptr = {m.ptr: m for m in self.meshes}

    def __del__(self):
        if getattr(self, "ptr", None):
            self._lib.vmh_visualmesh_destroy(self.ptr)
            self.ptr = None

    def height(self, h):
        return self._by_ptr[self._lib.vmh_visualmesh_height(self.ptr, float(h))]


class Engine:
    """visualmesh::engine::hip::Engine<float> for meshes of one model (0 = Ring6, 1 = NMGrid8)."""

    def __init__(self, network_groups, model, precision=native.FP32):
        self._lib = native.host()
        self.network = network_groups if isinstance(network_groups, Network) else Network(network_groups)
        self.model = model
        p = C.c_void_p()
        native.host_check(self._lib.vmh_engine_create(C.byref(self.network.c), model, precision, C.byref(p)))
        self.ptr = p
        self._staged = None

    def __del__(self):
        if getattr(self, "ptr", None):
            self._lib.vmh_engine_destroy(self.ptr)
            self.ptr = None

    @staticmethod
    def _pick(mesh, Hoc):
        return mesh.height(float(Hoc[2][3]))

    @staticmethod
    def _cap(mesh, Hoc, lens):
        r = mesh.lookup(Hoc, lens)
        return int((r[:, 1] - r[:, 0]).sum()) if len(r) else 0

    def project(self, mesh, Hoc, lens):
        m = self._pick(mesh, Hoc)
        H = np.ascontiguousarray(Hoc, dtype=np.float32)
        cap = self._cap(m, H, lens)
        px = np.zeros((max(cap, 1), 2), np.float32)
        nb = np.zeros((cap + 1, m.n_neighbours), np.int32)
        gidx = np.zeros(max(cap, 1), np.int32)
        V = native.host_check(self._lib.vmh_engine_project(self.ptr, m.ptr, _fp(H), C.byref(lens), cap, _fp(px), _ip(nb), _ip(gidx)))
        # nothing visible: the neighbourhood table is its null row alone, as the reference's projection returns it
        return dict(px=px[:V].copy(), nb=nb[:V + 1].copy(), gidx=gidx[:V].copy())

    def classify(self, mesh, Hoc, lens, image, fcc):
        m = self._pick(mesh, Hoc)
        H = np.ascontiguousarray(Hoc, dtype=np.float32)
        cap = self._cap(m, H, lens)
        n_out = self.network.n_out
        px = np.zeros((max(cap, 1), 2), np.float32)
        nb = np.zeros((cap + 1, m.n_neighbours), np.int32)
        gidx = np.zeros(max(cap, 1), np.int32)
        cls = np.zeros((cap + 1, n_out), np.float32)
        img = np.ascontiguousarray(image)
        V = native.host_check(self._lib.vmh_engine_classify(self.ptr, m.ptr, _fp(H), C.byref(lens), img.ctypes.data, fcc, cap,
                                                            _fp(px), _ip(nb), _ip(gidx), _fp(cls)))
        if V == 0:
            return dict(px=px[:0], nb=nb[:0], gidx=gidx[:0], cls=cls[:0])
        return dict(px=px[:V].copy(), nb=nb[:V + 1].copy(), gidx=gidx[:V].copy(), cls=cls[:V + 1].copy())

    def __call__(self, mesh, Hoc, lens, image=None, fcc=None):
        if image is None:
            return self.project(mesh, Hoc, lens)
        return self.classify(mesh, Hoc, lens, image, fcc)

    def time_calls(self, mesh, Hoc, lens, image, fcc, repeats=50):
        """(average milliseconds of one C++ call engine(mesh, Hoc, lens, image, fourcc) with its results returned by value,
        visible nodes): the calls are made and timed inside the C++ host library, one untimed call first"""
        m = self._pick(mesh, Hoc)
        H = np.ascontiguousarray(Hoc, dtype=np.float32)
        img = np.ascontiguousarray(image)
        ms = C.c_double(0.0)
        V = native.host_check(self._lib.vmh_engine_time_calls(self.ptr, m.ptr, _fp(H), C.byref(lens), img.ctypes.data, fcc, repeats, C.byref(ms)))
        return float(ms.value), V

    # ---- staged batches
    def stage(self, frames, wait=True):
        """frames: list of dict(mesh=Mesh|VisualMesh, Hoc, lens, image, fourcc); copies the inputs to the device.
        wait=False queues the copies ahead of the run and returns (Engine::stage_async): the images must then be
        page-locked (native.pinned_empty) and stay untouched until run() or wait() has returned."""
        n = len(frames)
        meshes = [self._pick(f["mesh"], f["Hoc"]) for f in frames]
        mesh_ptrs = (C.c_void_p * n)(*[m.ptr for m in meshes])
        H = np.ascontiguousarray(np.stack([np.asarray(f["Hoc"], dtype=np.float32) for f in frames]))
        lenses = (Lens * n)(*[f["lens"] for f in frames])
        images = [np.ascontiguousarray(f["image"]) for f in frames]
        image_ptrs = (C.c_void_p * n)(*[im.ctypes.data for im in images])
        fccs = (C.c_uint32 * n)(*[f["fourcc"] for f in frames])
        native.host_check(self._lib.vmh_engine_stage(self.ptr, n, mesh_ptrs, _fp(H), lenses, image_ptrs, fccs, int(bool(wait))))
        self._staged = meshes
        self._staged_images = images  # an asynchronous stage still reads them

    def run(self):
        native.host_check(self._lib.vmh_engine_run(self.ptr))

    def set_device_lookup(self, on=True):
        """stage() looks up the nodes that may be on screen on the device (same cone tree, same comparisons) instead of
        on the host"""
        self._lib.vmh_engine_set_device_lookup(self.ptr, int(bool(on)))

    def staged_ranges(self, index):
        """the lookup ranges of staged frame `index` as an [n, 2] array"""
        lib = native.hip()
        n = native.hip_check(lib.vmhip_batch_ranges(self.native_batch(), index, None, 0))
        out = np.zeros((max(n, 1), 2), np.int32)
        native.hip_check(lib.vmhip_batch_ranges(self.native_batch(), index, native._ip(out), n))
        return out[:n]

    def lookup_graph(self, index, same_edges=False):
        """Engine::lookup_graph of staged frame `index` (the training pipeline's LookupVisualMesh output): dict(vectors[n,3],
        graph[n,nn+1], px[n,2])"""
        nn = self._staged[index].n_neighbours
        n = native.host_check(self._lib.vmh_engine_lookup_graph(self.ptr, index, int(same_edges), 0, None, None, None))
        vectors, graph, px = np.zeros((n, 3), np.float32), np.zeros((n, nn + 1), np.int32), np.zeros((n, 2), np.float32)
        if n:
            native.host_check(self._lib.vmh_engine_lookup_graph(self.ptr, index, int(same_edges), n, _fp(vectors), _ip(graph), _fp(px)))
        return dict(vectors=vectors, graph=graph, px=px)

    def run_async(self):
        """launch the pass over the staged frames and return; wait() finishes it"""
        native.hip_check(native.hip().vmhip_batch_run_async(self.native_batch()))

    def wait(self):
        native.hip_check(native.hip().vmhip_batch_wait(self.native_batch()))

    def counts(self):
        n = len(self._staged)
        v = np.zeros(n, np.int32)
        native.host_check(self._lib.vmh_engine_counts(self.ptr, _ip(v), n))
        return v

    def fetch(self):
        n = native.host_check(self._lib.vmh_engine_fetch(self.ptr))
        counts = self.counts()
        out = []
        n_out = self.network.n_out
        for i in range(n):
            V = int(counts[i])
            m = self._staged[i]
            px = np.zeros((max(V, 1), 2), np.float32)
            nb = np.zeros((V + 1, m.n_neighbours), np.int32)
            gidx = np.zeros(max(V, 1), np.int32)
            cls = np.zeros((V + 1, n_out), np.float32)
            got = native.host_check(self._lib.vmh_engine_result(self.ptr, i, V, _fp(px), _ip(nb), _ip(gidx), _fp(cls)))
            assert got == V
            if V == 0:
                out.append(dict(px=px[:0], nb=nb[:0], gidx=gidx[:0], cls=cls[:0]))
            else:
                out.append(dict(px=px, nb=nb, gidx=gidx, cls=cls))
        return out

    def fetch_pinned(self, wait=True):
        """fetch() straight through the C ABI into page-locked arrays (vmhip_host_alloc), which the copies from the
        device reach at full PCIe speed and without a second copy on the host. The arrays belong to the engine and are
        reused by the next call. wait=False queues the copies and returns (vmhip_batch_fetch_async); fetch_wait() finishes
        them."""
        lib = native.hip()
        counts = self.counts()
        n = len(counts)
        n_out = self.network.n_out
        raw = (native.Result * n)()
        if not hasattr(self, "_pinned_results"):
            self._pinned_results = {}
        out = []
        for i in range(n):
            V = int(counts[i])
            nn = self._staged[i].n_neighbours
            held = self._pinned_results.get(i)
            if held is None or held["cap"] < V or held["nn"] != nn or held["n_out"] != n_out:
                cap = V + V // 8 + 1
                held = dict(cap=cap, nn=nn, n_out=n_out, px=native.pinned_empty((cap, 2), np.float32), nb=native.pinned_empty((cap + 1, nn), np.int32),
                            gidx=native.pinned_empty((cap,), np.int32), cls=native.pinned_empty((cap + 1, n_out), np.float32))
                self._pinned_results[i] = held
            raw[i] = native.Result(held["cap"], 0, _fp(held["px"]), _ip(held["gidx"]), _ip(held["nb"]), _fp(held["cls"]))
            out.append(dict(px=held["px"][:V], nb=held["nb"][:V + 1 if V else 0], gidx=held["gidx"][:V], cls=held["cls"][:V + 1 if V else 0]))
        if wait:
            native.hip_check(lib.vmhip_batch_fetch(self.native_batch(), raw))
        else:
            native.hip_check(lib.vmhip_batch_fetch_async(self.native_batch(), raw))
            self._raw_results = raw  # the copies read this table's pointers only at the call, but keep it with the arrays
        return out

    def fetch_packed(self, wait=True):
        """fetch_pinned() as one transfer (vmhip_batch_fetch_packed_async): a kernel gathers all frames' arrays into one block on
        the device and a single copy brings it into one page-locked block of the engine's; the arrays returned are views into
        it, valid after fetch_wait() (or at once with wait=True) and until the next fetch_packed()."""
        lib = native.hip()
        n = len(self._staged)
        need = int(lib.vmhip_batch_fetch_packed_size(self.native_batch()))
        block = getattr(self, "_packed_block", None)
        if block is None or block.nbytes < need:
            block = self._packed_block = native.pinned_empty((need + need // 8 + 256,), np.uint8)
        raw = (native.Result * n)()
        native.hip_check(lib.vmhip_batch_fetch_packed_async(self.native_batch(), block.ctypes.data, block.nbytes, raw))
        n_out = self.network.n_out
        out = []
        base = block.ctypes.data
        for i in range(n):
            V = raw[i].n_visible
            nn = self._staged[i].n_neighbours
            if V == 0:
                out.append(dict(px=np.zeros((0, 2), np.float32), nb=np.zeros((0, nn), np.int32), gidx=np.zeros(0, np.int32), cls=np.zeros((0, n_out), np.float32)))
                continue

            def view(pointer, count, dtype, shape):
                at = C.cast(pointer, C.c_void_p).value - base
                return block[at:at + count * 4].view(dtype).reshape(shape)

            out.append(dict(px=view(raw[i].pixel_coordinates, 2 * V, np.float32, (V, 2)), gidx=view(raw[i].global_indices, V, np.int32, (V,)),
                            nb=view(raw[i].neighbourhood, (V + 1) * nn, np.int32, (V + 1, nn)),
                            cls=view(raw[i].classifications, (V + 1) * n_out, np.float32, (V + 1, n_out))))
        self._raw_results = raw
        if wait:
            self.fetch_wait()
        return out

    def fetch_wait(self):
        """finishes fetch_pinned(wait=False): the arrays it returned are valid from here on"""
        native.hip_check(native.hip().vmhip_batch_fetch_wait(self.native_batch()))

    def classify_batch(self, frames):
        self.stage(frames)
        self.run()
        return self.fetch()

    def set_cache_limit(self, nbytes):
        self._lib.vmh_engine_set_cache_limit(self.ptr, int(nbytes))

    def cache_info(self):
        """(meshes resident on the device, their bytes)"""
        nbytes = C.c_uint64()
        n = self._lib.vmh_engine_cache_info(self.ptr, C.byref(nbytes))
        return n, nbytes.value

    def native_batch(self):
        return C.c_void_p(self._lib.vmh_engine_native_batch(self.ptr))

    def graph_stats(self):
        """dict(captures, graph_launches, eager_launches): how this engine's passes reached the stream so far"""
        return native.graph_stats(self.native_batch())

    def detect(self, class_index, threshold, arg_max_only=False, clusters=True):
        """The nodes of one class among the results of the last run, picked (probability >= threshold, optionally only
        where the class is the arg max) and grouped into connected components of the neighbourhood graph on the
        device; only they are downloaded. One dict per staged frame: node, pixel, probability, cluster,
        cluster_size, cluster_box, cluster_centre."""
        lib = native.hip()
        n = len(self._staged)
        raw = (native.Detections * n)()
        rc = lib.vmhip_batch_detect(self.native_batch(), class_index, threshold, int(arg_max_only), int(clusters), raw)
        out = []
        if rc == native.ERR_CAPACITY:  # the first call only counted
            for r in raw:
                d = dict(node=np.empty(r.n_detections, np.int32), pixel=np.empty((r.n_detections, 2), np.float32),
                         probability=np.empty(r.n_detections, np.float32),
                         cluster=np.empty(r.n_detections if clusters else 0, np.int32),
                         cluster_size=np.empty(r.n_clusters, np.int32), cluster_box=np.empty((r.n_clusters, 4), np.float32),
                         cluster_centre=np.empty((r.n_clusters, 2), np.float32))
                r.capacity, r.cluster_capacity = r.n_detections, r.n_clusters
                r.node, r.pixel, r.probability = native._ip(d["node"]), native._fp(d["pixel"]), native._fp(d["probability"])
                r.cluster = native._ip(d["cluster"]) if clusters else None
                r.cluster_size, r.cluster_box = native._ip(d["cluster_size"]), native._fp(d["cluster_box"])
                r.cluster_centre = native._fp(d["cluster_centre"])
                out.append(d)
            rc = lib.vmhip_batch_detect(self.native_batch(), class_index, threshold, int(arg_max_only), int(clusters), raw)
        else:
            out = [dict(node=np.empty(0, np.int32), pixel=np.empty((0, 2), np.float32), probability=np.empty(0, np.float32),
                        cluster=np.empty(0, np.int32), cluster_size=np.empty(0, np.int32),
                        cluster_box=np.empty((0, 4), np.float32), cluster_centre=np.empty((0, 2), np.float32)) for _ in range(n)]
        native.hip_check(rc)
        return out

    def profile(self, enable=True):
        """0/False off, 1/True every kernel, 2 only the kernel that took longest in the last fully profiled run"""
        if not self.native_batch():
            return  # nothing staged yet: profiling is switched on per batch object
        native.hip_check(native.hip().vmhip_batch_profile(self.native_batch(), int(enable)))

    def profile_read(self):
        return native.profile_read(self.native_batch())


class Pipeline:
    """visualmesh::engine::hip::Pipeline<float>: three engines in rotation behind one submit() call. submit(frames) queues a
    batch (images in page-locked memory, untouched until the next call returns) and returns the results of the batch
    submitted two calls earlier, or None while the pipeline fills; flush() drains (None when empty). The arrays returned
    are views into the pipeline's page-locked memory, valid until two more calls."""

    def __init__(self, network_groups, model, precision=native.FP32):
        self._lib = native.host()
        self.network = network_groups if isinstance(network_groups, Network) else Network(network_groups)
        self.model = model
        p = C.c_void_p()
        native.host_check(self._lib.vmh_pipeline_create(C.byref(self.network.c), model, precision, C.byref(p)))
        self.ptr = p
        self._neighbours = []   # per batch in flight: the frames' neighbour counts
        self._keep = []         # per batch in flight: what the asynchronous stage still reads

    def __del__(self):
        if getattr(self, "ptr", None):
            self._lib.vmh_pipeline_destroy(self.ptr)
            self.ptr = None

    def _results(self, n_done, arrays=True):
        if n_done == 0:
            return None
        nns = self._neighbours.pop(0)
        self._keep.pop(0)
        if not arrays:
            return n_done
        n_out = self.network.n_out
        out = []
        for i in range(n_done):
            px, gidx, nb, cls = C.POINTER(C.c_float)(), C.POINTER(C.c_int32)(), C.POINTER(C.c_int32)(), C.POINTER(C.c_float)()
            V = native.host_check(self._lib.vmh_pipeline_result(self.ptr, i, C.byref(px), C.byref(gidx), C.byref(nb), C.byref(cls)))
            nn = nns[i]
            if V == 0:
                out.append(dict(px=np.zeros((0, 2), np.float32), nb=np.zeros((0, nn), np.int32), gidx=np.zeros(0, np.int32), cls=np.zeros((0, n_out), np.float32)))
                continue
            out.append(dict(px=np.ctypeslib.as_array(px, (V, 2)), gidx=np.ctypeslib.as_array(gidx, (V,)),
                            nb=np.ctypeslib.as_array(nb, (V + 1, nn)), cls=np.ctypeslib.as_array(cls, (V + 1, n_out))))
        return out

    def submit(self, frames, arrays=True):
        """arrays=False: the number of frames of the finished batch instead of numpy views of its results (a caller that
        only counts, like a benchmark loop, saves the time numpy takes to wrap 4 arrays per frame)"""
        n = len(frames)
        meshes = [f["mesh"].height(float(f["Hoc"][2][3])) for f in frames]
        mesh_ptrs = (C.c_void_p * n)(*[m.ptr for m in meshes])
        H = np.ascontiguousarray(np.stack([np.asarray(f["Hoc"], dtype=np.float32) for f in frames]))
        lenses = (Lens * n)(*[f["lens"] for f in frames])
        images = [np.ascontiguousarray(f["image"]) for f in frames]
        image_ptrs = (C.c_void_p * n)(*[im.ctypes.data for im in images])
        fccs = (C.c_uint32 * n)(*[f["fourcc"] for f in frames])
        self._neighbours.append([m.n_neighbours for m in meshes])
        self._keep.append(images)
        return self._results(native.host_check(self._lib.vmh_pipeline_submit(self.ptr, n, mesh_ptrs, _fp(H), lenses, image_ptrs, fccs)), arrays)

    def graph_stats(self):
        """dict(captures, graph_launches, eager_launches) of the three engines together"""
        v = [C.c_int64(0) for _ in range(3)]
        native.host_check(self._lib.vmh_pipeline_graph_stats(self.ptr, *[C.byref(x) for x in v]))
        return dict(captures=v[0].value, graph_launches=v[1].value, eager_launches=v[2].value)

    def flush(self, arrays=True):
        if not self._neighbours:
            return None
        return self._results(native.host_check(self._lib.vmh_pipeline_submit(self.ptr, 0, None, None, None, None, None)), arrays)


def load_model(path):
    """An exported model file through the C++ reader (visualmesh::load_model_file): dict(mesh, shape, radius,
    intersections, network) with network = list of groups of (weights[n_in, n_out], biases[n_out], activation)."""
    lib = native.host()
    handle = lib.vmh_model_load(str(path).encode())
    if not handle:
        raise RuntimeError("load_model: " + lib.vmh_last_error().decode())
    try:
        mesh = C.create_string_buffer(64)
        shape = C.create_string_buffer(64)
        radius, intersections = C.c_float(), C.c_float()
        n_groups = native.host_check(lib.vmh_model_info(handle, mesh, shape, 64, C.byref(radius), C.byref(intersections)))
        network = []
        for g in range(n_groups):
            group = []
            for l in range(native.host_check(lib.vmh_model_group_size(handle, g))):
                n_in, n_out, act = C.c_int(), C.c_int(), C.c_int()
                native.host_check(lib.vmh_model_layer(handle, g, l, C.byref(n_in), C.byref(n_out), C.byref(act), None, None))
                w = np.zeros((n_in.value, n_out.value), np.float32)
                b = np.zeros(n_out.value, np.float32)
                native.host_check(lib.vmh_model_layer(handle, g, l, C.byref(n_in), C.byref(n_out), C.byref(act), _fp(w), _fp(b)))
                group.append((w, b, act.value))
            network.append(group)
        return dict(mesh=mesh.value.decode(), shape=shape.value.decode(), radius=radius.value,
                    intersections=intersections.value, network=network)
    finally:
        lib.vmh_model_free(handle)


def load_lens(path, width, height):
    """One dataset lens file through the C++ reader: (Lens, Hoc[4, 4] float32)."""
    lib = native.host()
    lens = Lens()
    Hoc = np.zeros((4, 4), np.float32)
    native.host_check(lib.vmh_lens_load(str(path).encode(), width, height, C.byref(lens), _fp(Hoc)))
    return lens, Hoc


# ---------------------------------------------------------------------------------------------- Scalar = double
def _dp(a):
    return a.ctypes.data_as(C.POINTER(C.c_double))


class Mesh64:
    """Mesh<double, Model> of the C++ host code"""

    def __init__(self, model=None, shape=None, radius=None, h=None, k=None, max_distance=None, _ptr=None):
        self._lib = native.host64()
        self._owned = _ptr is None
        if _ptr is None:
            _ptr = self._lib.vmh_mesh_create(model, shape, radius, h, k, max_distance)
            if not _ptr:
                raise RuntimeError("mesh construction failed: " + self._lib.vmh_last_error().decode())
        self.ptr = _ptr
        self.n_nodes = self._lib.vmh_mesh_n_nodes(_ptr)
        self.n_neighbours = self._lib.vmh_mesh_n_neighbours(_ptr)
        self.h = self._lib.vmh_mesh_h(_ptr)
        self._arrays = None

    def __del__(self):
        if getattr(self, "_owned", False) and self.ptr:
            self._lib.vmh_mesh_destroy(self.ptr)
            self.ptr = None

    def arrays(self):
        """(rays[n,3] float64, neighbours[n,nn] int32) in mesh order"""
        if self._arrays is None:
            rays = np.zeros((self.n_nodes, 3), np.float64)
            nbr = np.zeros((self.n_nodes, self.n_neighbours), np.int32)
            self._lib.vmh_mesh_copy(self.ptr, _dp(rays), _ip(nbr))
            self._arrays = (rays, nbr)
        return self._arrays

    def lookup(self, Hoc, lens):
        H = np.ascontiguousarray(Hoc, dtype=np.float64)
        cap = 4096
        while True:
            r = np.zeros((cap, 2), np.int32)
            n = native.host_check(self._lib.vmh_mesh_lookup(self.ptr, _dp(H), C.byref(lens), _ip(r), cap), self._lib)
            if n <= cap:
                return r[:n].copy()
            cap = n

    def height(self, h):
        return self


class VisualMesh64:
    """VisualMesh<double, Model> of the C++ host code"""

    def __init__(self, model, shape, radius, min_h, max_h, k, max_error, max_distance):
        self._lib = native.host64()
        self.ptr = self._lib.vmh_visualmesh_create(model, shape, radius, min_h, max_h, k, max_error, max_distance)
        if not self.ptr:
            raise RuntimeError("visual mesh construction failed: " + self._lib.vmh_last_error().decode())
        n = self._lib.vmh_visualmesh_n_meshes(self.ptr)
        self.meshes = [Mesh64(_ptr=self._lib.vmh_visualmesh_mesh(self.ptr, i)) for i in range(n)]
        self._by_ptr = {m.ptr: m for m in self.meshes}

    def __del__(self):
        if getattr(self, "ptr", None):
            self._lib.vmh_visualmesh_destroy(self.ptr)
            self.ptr = None

    def height(self, h):
        return self._by_ptr[self._lib.vmh_visualmesh_height(self.ptr, float(h))]


class Engine64:
    """visualmesh::engine::hip::Engine<double> for meshes of one model (0 = Ring6, 1 = NMGrid8)."""

    def __init__(self, network_groups, model):
        self._lib = native.host64()
        self.network = network_groups if isinstance(network_groups, native.Network64) else native.Network64(network_groups)
        self.model = model
        p = C.c_void_p()
        native.host_check(self._lib.vmh_engine_create(C.byref(self.network.c), model, native.FP64, C.byref(p)), self._lib)
        self.ptr = p

    def __del__(self):
        if getattr(self, "ptr", None):
            self._lib.vmh_engine_destroy(self.ptr)
            self.ptr = None

    def _buffers(self, mesh, Hoc, lens):
        m = mesh.height(float(Hoc[2][3]))
        H = np.ascontiguousarray(Hoc, dtype=np.float64)
        r = m.lookup(H, lens)
        cap = int((r[:, 1] - r[:, 0]).sum()) if len(r) else 0
        return m, H, cap, np.zeros((max(cap, 1), 2), np.float64), np.zeros((cap + 1, m.n_neighbours), np.int32), np.zeros(max(cap, 1), np.int32)

    def project(self, mesh, Hoc, lens):
        m, H, cap, px, nb, gidx = self._buffers(mesh, Hoc, lens)
        V = native.host_check(self._lib.vmh_engine_project(self.ptr, m.ptr, _dp(H), C.byref(lens), cap, _dp(px), _ip(nb), _ip(gidx)), self._lib)
        return dict(px=px[:V].copy(), nb=nb[:V + 1].copy(), gidx=gidx[:V].copy())

    def classify(self, mesh, Hoc, lens, image, fcc):
        m, H, cap, px, nb, gidx = self._buffers(mesh, Hoc, lens)
        cls = np.zeros((cap + 1, self.network.n_out), np.float64)
        img = np.ascontiguousarray(image)
        V = native.host_check(self._lib.vmh_engine_classify(self.ptr, m.ptr, _dp(H), C.byref(lens), img.ctypes.data, fcc, cap,
                                                            _dp(px), _ip(nb), _ip(gidx), _dp(cls)), self._lib)
        if V == 0:
            return dict(px=px[:0], nb=nb[:0], gidx=gidx[:0], cls=cls[:0])
        return dict(px=px[:V].copy(), nb=nb[:V + 1].copy(), gidx=gidx[:V].copy(), cls=cls[:V + 1].copy())

    def __call__(self, mesh, Hoc, lens, image=None, fcc=None):
        if image is None:
            return self.project(mesh, Hoc, lens)
        return self.classify(mesh, Hoc, lens, image, fcc)

    def guard_stats(self):
        """dict(listed, overruled): near-edge nodes the device listed, device decisions the host overruled"""
        a, b = C.c_int64(0), C.c_int64(0)
        native.host_check(self._lib.vmh_engine_guard_stats(self.ptr, C.byref(a), C.byref(b)), self._lib)
        return dict(listed=a.value, overruled=b.value)

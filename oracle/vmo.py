"""ctypes binding of the CPU oracle's C interface (vm_oracle.h).

TEST INFRASTRUCTURE ONLY: imported by tests/, by bench.py's cpu_baseline leg and by
__graft_entry__.smoke(); never by the engine package.

`load("oracle")` opens libvm_oracle.so (the restatement), `load("reference")` opens
_ref/libvm_ref.so (the reference's own headers behind the same interface) and returns None when that
library has not been built.
"""
import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))

RING6, NMGRID8 = 0, 1
SPHERE, CIRCLE = 0, 1
RECTILINEAR, EQUISOLID, EQUIDISTANT = 0, 1, 2
SELU, RELU, SOFTMAX, TANH = 0, 1, 2, 3
ERR_FORMAT, ERR_LENS, ERR_ARG, ERR_CAPACITY = -2, -3, -4, -5


def fourcc(s):
    b = s.encode()
    assert len(b) == 4
    return b[0] | (b[1] << 8) | (b[2] << 16) | (b[3] << 24)


def _make_types(creal):
    """(Lens, _Layer, _Network) of vm_oracle.h for one vmo_real"""

    class Lens(C.Structure):
        _fields_ = [
            ("width", C.c_int32),
            ("height", C.c_int32),
            ("projection", C.c_int32),
            ("focal_length", creal),
            ("centre", creal * 2),
            ("k", creal * 2),
            ("fov", creal),
        ]

    class _Layer(C.Structure):
        _fields_ = [
            ("n_in", C.c_int32),
            ("n_out", C.c_int32),
            ("activation", C.c_int32),
            ("weights", C.POINTER(creal)),
            ("biases", C.POINTER(creal)),
        ]

    class _Network(C.Structure):
        _fields_ = [("n_groups", C.c_int32), ("group_sizes", C.POINTER(C.c_int32)), ("layers", C.POINTER(_Layer))]

    return Lens, _Layer, _Network


_TYPES = {"f32": (C.c_float, np.float32) + _make_types(C.c_float), "f64": (C.c_double, np.float64) + _make_types(C.c_double)}
Lens = _TYPES["f32"][2]


def make_lens(width, height, projection, focal_length, fov, centre=(0.0, 0.0), k=(0.0, 0.0), real="f32"):
    creal, _, lens_t = _TYPES[real][:3]
    return lens_t(width, height, projection, focal_length, (creal * 2)(*centre), (creal * 2)(*k), fov)


def _ip(a):
    return a.ctypes.data_as(C.POINTER(C.c_int32))


class Network:
    """network = list of groups, group = list of (weights[n_in, n_out], biases[n_out], activation); real picks the
    library the network is for: "f32" (float) or "f64" (double)."""

    def __init__(self, groups, real="f32"):
        creal, dtype, _, layer_t, network_t = _TYPES[real]
        self.groups = groups
        self.real = real
        self._keep = []
        layers = []
        for g in groups:
            for (w, b, act) in g:
                w = np.ascontiguousarray(w, dtype=dtype)
                b = np.ascontiguousarray(b, dtype=dtype)
                self._keep += [w, b]
                layers.append(layer_t(w.shape[0], w.shape[1], act, w.ctypes.data_as(C.POINTER(creal)),
                                      b.ctypes.data_as(C.POINTER(creal))))
        self._layers = (layer_t * max(len(layers), 1))(*layers)
        self._sizes = (C.c_int32 * max(len(groups), 1))(*[len(g) for g in groups])
        self.c = network_t(len(groups), self._sizes, self._layers)
        self.n_out = groups[-1][-1][0].shape[1] if groups else 4


class Oracle:
    def __init__(self, path, real="f32"):
        self.lib = L = C.CDLL(path)
        self.real = real
        self.creal, self.dtype, Lens, _Layer, _Network = _TYPES[real]
        creal = self.creal
        vp = C.c_void_p
        L.vmo_name.restype = C.c_char_p
        L.vmo_mesh_create.restype = vp
        L.vmo_mesh_create.argtypes = [C.c_int, C.c_int, creal, creal, creal, creal]
        L.vmo_mesh_destroy.argtypes = [vp]
        L.vmo_mesh_n_nodes.argtypes = [vp]
        L.vmo_mesh_n_neighbours.argtypes = [vp]
        L.vmo_mesh_h.argtypes = [vp]
        L.vmo_mesh_h.restype = creal
        L.vmo_mesh_copy.argtypes = [vp, C.POINTER(creal), C.POINTER(C.c_int32)]
        L.vmo_mesh_lookup.argtypes = [vp, C.POINTER(creal), C.POINTER(Lens), C.POINTER(C.c_int32), C.c_int]
        L.vmo_visualmesh_create.restype = vp
        L.vmo_visualmesh_create.argtypes = [C.c_int, C.c_int] + [creal] * 6
        L.vmo_visualmesh_destroy.argtypes = [vp]
        L.vmo_visualmesh_n_meshes.argtypes = [vp]
        L.vmo_visualmesh_mesh.restype = vp
        L.vmo_visualmesh_mesh.argtypes = [vp, C.c_int]
        L.vmo_visualmesh_height.restype = vp
        L.vmo_visualmesh_height.argtypes = [vp, creal]
        L.vmo_project.argtypes = [vp, C.POINTER(creal), C.POINTER(Lens), C.c_int, C.POINTER(creal),
                                  C.POINTER(C.c_int32), C.POINTER(C.c_int32)]
        L.vmo_classify.argtypes = [vp, C.POINTER(creal), C.POINTER(Lens), vp, C.c_uint32, C.POINTER(_Network),
                                   C.c_int, C.POINTER(creal), C.POINTER(C.c_int32), C.POINTER(C.c_int32),
                                   C.POINTER(creal)]
        L.vmo_fn_project.argtypes = [C.POINTER(creal), C.POINTER(Lens), C.POINTER(creal)]
        L.vmo_fn_unproject.argtypes = [C.POINTER(creal), C.POINTER(Lens), C.POINTER(creal)]
        L.vmo_fn_interpolate.argtypes = [C.POINTER(creal), vp, C.c_int, C.c_int, C.c_uint32, C.POINTER(creal)]
        L.vmo_fn_get_pixel.argtypes = [C.c_int, C.c_int, vp, C.c_int, C.c_int, C.c_uint32, C.POINTER(creal)]
        L.vmo_fn_activation.argtypes = [C.c_int, C.POINTER(creal), C.c_int, C.c_int]
        L.vmo_fn_shape.restype = creal
        L.vmo_fn_shape.argtypes = [C.c_int, creal, C.c_int, creal, creal]
        L.vmo_fn_libm.argtypes = [C.c_int, C.POINTER(creal), C.POINTER(creal), C.c_int]
        self.name = L.vmo_name().decode()

    def _fp(self, a):
        assert a.dtype == self.dtype
        return a.ctypes.data_as(C.POINTER(self.creal))

    def make_lens(self, *args, **kw):
        return make_lens(*args, real=self.real, **kw)

    def network(self, groups):
        return Network(groups, real=self.real)

    # ---- meshes
    def mesh(self, model, shape, radius, h, k, max_distance):
        p = self.lib.vmo_mesh_create(model, shape, radius, h, k, max_distance)
        if not p:
            raise RuntimeError("mesh construction failed")
        return Mesh(self, p, owned=True)

    def visualmesh(self, model, shape, radius, min_h, max_h, k, max_error, max_distance):
        p = self.lib.vmo_visualmesh_create(model, shape, radius, min_h, max_h, k, max_error, max_distance)
        if not p:
            raise RuntimeError("visual mesh construction failed")
        return VisualMesh(self, p)

    # ---- single functions
    def fn_project(self, ray, lens):
        r = np.asarray(ray, dtype=self.dtype)
        o = np.zeros(2, self.dtype)
        self.lib.vmo_fn_project(self._fp(r), C.byref(lens), self._fp(o))
        return o

    def fn_unproject(self, px, lens):
        p = np.asarray(px, dtype=self.dtype)
        o = np.zeros(3, self.dtype)
        self.lib.vmo_fn_unproject(self._fp(p), C.byref(lens), self._fp(o))
        return o

    def fn_interpolate(self, px, image, width, height, fcc):
        p = np.asarray(px, dtype=self.dtype)
        o = np.zeros(4, self.dtype)
        rc = self.lib.vmo_fn_interpolate(self._fp(p), image.ctypes.data, width, height, fcc, self._fp(o))
        if rc != 0:
            raise ValueError("unsupported format (%d)" % rc)
        return o

    def fn_get_pixel(self, x, y, image, width, height, fcc):
        o = np.zeros(4, self.dtype)
        rc = self.lib.vmo_fn_get_pixel(x, y, image.ctypes.data, width, height, fcc, self._fp(o))
        if rc != 0:
            raise ValueError("unsupported format (%d)" % rc)
        return o

    def fn_activation(self, act, data, dims):
        d = np.ascontiguousarray(data, dtype=self.dtype).copy()
        self.lib.vmo_fn_activation(act, self._fp(d), d.size // dims, dims)
        return d

    def fn_libm(self, which, x):
        """host libm: which in acos, sin, tan, sqrt"""
        x = np.ascontiguousarray(x, dtype=self.dtype)
        y = np.zeros_like(x)
        self.lib.vmo_fn_libm({"acos": 0, "sin": 1, "tan": 2, "sqrt": 3}[which], self._fp(x), self._fp(y), x.size)
        return y

    def fn_shape(self, shape, radius, which, a=0.0, b=0.0):
        return self.lib.vmo_fn_shape(shape, radius, {"phi": 0, "n": 1, "theta": 2, "k": 3, "c": 4}[which], a, b)


class Mesh:
    def __init__(self, oracle, ptr, owned):
        self.o, self.ptr, self.owned = oracle, ptr, owned
        L = oracle.lib
        self.n_nodes = L.vmo_mesh_n_nodes(ptr)
        self.n_neighbours = L.vmo_mesh_n_neighbours(ptr)
        self.h = L.vmo_mesh_h(ptr)
        self._arrays = None

    def __del__(self):
        if self.owned and self.ptr:
            self.o.lib.vmo_mesh_destroy(self.ptr)
            self.ptr = None

    def arrays(self):
        """(rays[n,3] float32, neighbours[n,nn] int32)"""
        if self._arrays is None:
            rays = np.zeros((self.n_nodes, 3), self.o.dtype)
            nbr = np.zeros((self.n_nodes, self.n_neighbours), np.int32)
            self.o.lib.vmo_mesh_copy(self.ptr, self.o._fp(rays), _ip(nbr))
            self._arrays = (rays, nbr)
        return self._arrays

    def lookup(self, Hoc, lens):
        H = np.ascontiguousarray(Hoc, dtype=self.o.dtype)
        cap = 4096
        while True:
            r = np.zeros((cap, 2), np.int32)
            n = self.o.lib.vmo_mesh_lookup(self.ptr, self.o._fp(H), C.byref(lens), _ip(r), cap)
            if n < 0:
                raise RuntimeError("lookup failed (%d)" % n)
            if n <= cap:
                return r[:n].copy()
            cap = n

    def lookup_graph(self, Hoc, lens, same_edges=False):
        """What the training pipeline's LookupVisualMesh op returns, restated from the reference's
        tensorflow/lookup.cpp:186-249 (that file needs TensorFlow's headers and cannot be compiled here; the reference
        holds no test or fixture of the op, so tests pin this restatement by the graph's own invariants instead):
        vectors[n,3] = the unit vectors of the nodes in the lookup ranges, in order; graph[n,nn+1] = own position, then
        the neighbours' positions along the ranges through a reverse table that starts out as the most negative int32
        (lookup.cpp:207-216, 231-235). same_edges applies training/dataset/projection/visual_mesh.py:86-87:
        negative entries become the row's first column. -> dict(vectors, graph, gidx)"""
        rays, nbr = self.arrays()
        ranges = self.lookup(Hoc, lens)
        gidx = np.concatenate([np.arange(a, b, dtype=np.int64) for a, b in ranges]) if len(ranges) else np.zeros(0, np.int64)
        r_lookup = np.full(self.n_nodes + 1, np.iinfo(np.int32).min, np.int32)
        r_lookup[gidx] = np.arange(len(gidx), dtype=np.int32)
        graph = np.concatenate([np.arange(len(gidx), dtype=np.int32)[:, None], r_lookup[nbr[gidx]]], axis=1)
        if same_edges:
            graph = np.where(graph < 0, graph[:, :1], graph)
        return dict(vectors=rays[gidx].copy(), graph=graph.astype(np.int32), gidx=gidx.astype(np.int32))

    def project(self, Hoc, lens):
        """-> dict(px[V,2], nb[V+1,nn], gidx[V])"""
        H = np.ascontiguousarray(Hoc, dtype=self.o.dtype)
        ranges = self.lookup(Hoc, lens)
        cap = int((ranges[:, 1] - ranges[:, 0]).sum()) if len(ranges) else 0
        px = np.zeros((max(cap, 1), 2), self.o.dtype)
        nb = np.zeros((cap + 1, self.n_neighbours), np.int32)
        gidx = np.zeros(max(cap, 1), np.int32)
        V = self.o.lib.vmo_project(self.ptr, self.o._fp(H), C.byref(lens), cap, self.o._fp(px), _ip(nb), _ip(gidx))
        if V < 0:
            raise RuntimeError("project failed (%d)" % V)
        return dict(px=px[:V].copy(), nb=nb[:V + 1].copy(), gidx=gidx[:V].copy(), ranges=ranges)

    def classify(self, Hoc, lens, image, fcc, network):
        """-> dict(px, nb, gidx, cls[V+1, n_out]); an empty visible set gives empty arrays (default result)"""
        H = np.ascontiguousarray(Hoc, dtype=self.o.dtype)
        ranges = self.lookup(Hoc, lens)
        cap = int((ranges[:, 1] - ranges[:, 0]).sum()) if len(ranges) else 0
        n_out = network.n_out
        px = np.zeros((max(cap, 1), 2), self.o.dtype)
        nb = np.zeros((cap + 1, self.n_neighbours), np.int32)
        gidx = np.zeros(max(cap, 1), np.int32)
        cls = np.zeros((cap + 1, n_out), self.o.dtype)
        img = np.ascontiguousarray(image)
        V = self.o.lib.vmo_classify(self.ptr, self.o._fp(H), C.byref(lens), img.ctypes.data, fcc, C.byref(network.c), cap,
                                    self.o._fp(px), _ip(nb), _ip(gidx), self.o._fp(cls))
        if V == ERR_FORMAT:
            raise ValueError("Unsupported image format")
        if V < 0:
            raise RuntimeError("classify failed (%d)" % V)
        if V == 0:
            return dict(px=px[:0], nb=nb[:0], gidx=gidx[:0], cls=cls[:0], ranges=ranges)
        return dict(px=px[:V].copy(), nb=nb[:V + 1].copy(), gidx=gidx[:V].copy(), cls=cls[:V + 1].copy(), ranges=ranges)


class VisualMesh:
    def __init__(self, oracle, ptr):
        self.o, self.ptr = oracle, ptr
        n = oracle.lib.vmo_visualmesh_n_meshes(ptr)
        self.meshes = [Mesh(oracle, oracle.lib.vmo_visualmesh_mesh(ptr, i), owned=False) for i in range(n)]
        self._by_ptr = {m.ptr: m for m in self.meshes}

    def __del__(self):
        if self.ptr:
            self.o.lib.vmo_visualmesh_destroy(self.ptr)
            self.ptr = None

    def height(self, h):
        return self._by_ptr[self.o.lib.vmo_visualmesh_height(self.ptr, h)]


_cache = {}


def load(which="oracle", real="f32"):
    """which: "oracle" (the restatement) or "reference" (the reference's headers; None where that library is not
    built); real: "f32" for Scalar = float, "f64" for Scalar = double"""
    key = (which, real)
    if key not in _cache:
        suffix = "" if real == "f32" else "_f64"
        path = (os.path.join(HERE, "libvm_oracle%s.so" % suffix) if which == "oracle"
                else os.path.join(HERE, "_ref", "libvm_ref%s.so" % suffix))
        if not os.path.exists(path):
            if which == "oracle":
                raise FileNotFoundError(path + " is not built: run `make -C oracle` or __graft_entry__.build()")
            _cache[key] = None
        else:
            _cache[key] = Oracle(path, real)
    return _cache[key]

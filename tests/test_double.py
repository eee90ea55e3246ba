"""Scalar = double: the reference's engines and meshes are templates over Scalar (engine/cpu/engine.hpp:49-50,
mesh.hpp:56; the training op registers float and double, tensorflow/lookup.cpp:255-278). The restatement compiled for
double (oracle/libvm_oracle_f64.so) against the reference's own headers instantiated with double
(oracle/_ref/libvm_ref_f64.so): bit equality of every stage. Skipped where the reference tree was not mounted at build
time."""
import math

import numpy as np
import pytest

from helpers import bits_equal
from visualmesh_amd import workloads as wl


def _cmp_all(a, b, keys):
    for k in keys:
        assert a[k].dtype == b[k].dtype and bits_equal(a[k], b[k]), k


def network64(groups):
    return [[(w.astype(np.float64), b.astype(np.float64), act) for (w, b, act) in g] for g in groups]


@pytest.mark.parametrize("args", [
    (wl.RING6, wl.SPHERE, 0.0949, 1.2, 6.0, 20.0),
    (wl.RING6, wl.CIRCLE, 0.05, 0.9, 5.0, 4.0),
    (wl.NMGRID8, wl.CIRCLE, 0.05, 1.2, 8.0, 2.0),
    (wl.NMGRID8, wl.SPHERE, 0.0949, 1.0, 4.0, 5.0),
])
def test_mesh_lookup_projection(oracle64, reference64, args):
    a, b = oracle64.mesh(*args), reference64.mesh(*args)
    assert a.n_nodes == b.n_nodes
    assert a.arrays()[0].dtype == np.float64
    assert bits_equal(a.arrays()[0], b.arrays()[0]) and bits_equal(a.arrays()[1], b.arrays()[1])
    rng = np.random.default_rng(3)
    for (W, H, proj, f, fov) in [(1280, 1024, wl.EQUISOLID, 420.0, math.pi), (1280, 1024, wl.RECTILINEAR, 700.0, math.pi / 2),
                                 (2048, 1536, wl.EQUIDISTANT, 672.0, math.pi)]:
        for i in range(5):
            k = (0.0, 0.0) if i < 4 else (-1.0e-7, 2.0e-14)
            lens = oracle64.make_lens(W, H, proj, f, fov, centre=(float(rng.uniform(-10, 10)), float(rng.uniform(-10, 10))), k=k)
            Hoc = wl.make_hoc(args[3], math.radians(rng.uniform(-20, 100)), math.radians(rng.uniform(-20, 20)),
                              math.radians(rng.uniform(-180, 180)), dtype=np.float64)
            _cmp_all(a.project(Hoc, lens), b.project(Hoc, lens), ("ranges", "px", "nb", "gidx"))


def test_the_double_mesh_is_not_the_float_mesh(oracle, oracle64):
    """the two Scalars give different meshes (ring sizes come from ceil() of quotients): a double engine fed a float
    mesh, or the other way round, would not be the reference's"""
    args = (wl.RING6, wl.SPHERE, 0.0949, 1.2, 6.0, 20.0)
    a, b = oracle.mesh(*args), oracle64.mesh(*args)
    ra, rb = a.arrays()[0], b.arrays()[0]
    assert ra.dtype == np.float32 and rb.dtype == np.float64
    assert a.n_nodes != b.n_nodes or not np.array_equal(ra.astype(np.float64), rb)


@pytest.mark.parametrize("index", [1, 3])
def test_classification_of_configs(oracle64, reference64, index):
    cfg = wl.config(index)
    args = (cfg.model, cfg.shape, cfg.radius, cfg.mesh_h, cfg.k, min(cfg.max_distance, 3.0) if index == 3 else cfg.max_distance)
    a, b = oracle64.mesh(*args), reference64.mesh(*args)
    lens = oracle64.make_lens(*cfg.lens_tuple())
    f = cfg.frames[0]
    net = oracle64.network(network64(cfg.network))
    Hoc = f["Hoc"].astype(np.float64)
    _cmp_all(a.classify(Hoc, lens, f["image"], cfg.fourcc, net), b.classify(Hoc, lens, f["image"], cfg.fourcc, net),
             ("ranges", "px", "nb", "gidx", "cls"))


@pytest.mark.parametrize("code", ["RGBA", "BGRA", "RGB3", "BGR8", "GRAY", "Y8  ", "GRBG", "RGGB", "GBRG", "BGGR"])
def test_every_pixel_format(oracle64, reference64, code):
    rng = np.random.default_rng(9)
    W, H = 64, 48
    bpp = {"RGBA": 4, "BGRA": 4, "RGB3": 3, "BGR8": 3}.get(code, 1)
    img = wl.random_image(rng, W, H, bpp)
    fcc = wl.fourcc(code)
    for _ in range(300):
        px = (float(rng.uniform(0, W - 1.001)), float(rng.uniform(0, H - 1.001)))
        assert bits_equal(oracle64.fn_interpolate(px, img, W, H, fcc), reference64.fn_interpolate(px, img, W, H, fcc))
    for (x, y) in [(0, 0), (W - 1, 0), (0, H - 1), (W - 1, H - 1), (1, 1), (2, 5)]:
        assert bits_equal(oracle64.fn_get_pixel(x, y, img, W, H, fcc), reference64.fn_get_pixel(x, y, img, W, H, fcc))


def test_multi_layer_groups_and_all_activations(oracle64, reference64):
    rng = np.random.default_rng(21)
    args = (wl.RING6, wl.SPHERE, 0.0949, 1.0, 3.0, 8.0)
    a, b = oracle64.mesh(*args), reference64.mesh(*args)
    groups = [
        [(rng.normal(0, 0.3, (28, 8)), rng.normal(0, 0.1, 8), wl.TANH), (rng.normal(0, 0.3, (8, 6)), rng.normal(0, 0.1, 6), wl.RELU)],
        [(rng.normal(0, 0.3, (42, 5)), rng.normal(0, 0.1, 5), wl.SELU), (rng.normal(0, 0.3, (5, 3)), rng.normal(0, 0.1, 3), wl.SOFTMAX)],
    ]
    lens = oracle64.make_lens(320, 256, wl.EQUISOLID, 105.0, math.pi)
    Hoc = wl.make_hoc(1.0, math.radians(35), 0.03, -0.02, dtype=np.float64)
    img = wl.random_image(rng, 320, 256, 4)
    net = oracle64.network(groups)
    _cmp_all(a.classify(Hoc, lens, img, wl.fourcc("RGBA"), net), b.classify(Hoc, lens, img, wl.fourcc("RGBA"), net),
             ("px", "nb", "gidx", "cls"))


def test_visualmesh(oracle64, reference64):
    args = (wl.RING6, wl.SPHERE, 0.0949, 0.8, 1.5, 6.0, 0.5, 20.0)
    a, b = oracle64.visualmesh(*args), reference64.visualmesh(*args)
    assert [m.h for m in a.meshes] == [m.h for m in b.meshes]
    for ma, mb in zip(a.meshes, b.meshes):  # every height: sin/cos of other arguments than the single meshes above
        assert bits_equal(ma.arrays()[0], mb.arrays()[0]) and bits_equal(ma.arrays()[1], mb.arrays()[1])
    for h in np.linspace(0.6, 1.7, 45):
        assert a.height(float(h)).h == b.height(float(h)).h


def test_shape_functions(oracle64, reference64):
    rng = np.random.default_rng(1)
    for shape in (wl.SPHERE, wl.CIRCLE):
        for _ in range(500):
            r, h = float(rng.uniform(0.02, 0.2)), float(rng.uniform(0.5, 2.0))
            n = float(rng.uniform(0, 60))
            for which, x, y in (("phi", n, h), ("theta", n, h), ("n", float(rng.uniform(0.01, 1.5)), h), ("k", h, h * 1.1), ("c", 0, 0)):
                va, vb = oracle64.fn_shape(shape, r, which, x, y), reference64.fn_shape(shape, r, which, x, y)
                assert np.float64(va).view(np.uint64) == np.float64(vb).view(np.uint64) or (va != va and vb != vb)


def test_single_functions(oracle64, reference64):
    rng = np.random.default_rng(5)
    for proj, f, fov in ((wl.EQUISOLID, 420.0, math.pi), (wl.RECTILINEAR, 700.0, math.pi / 2), (wl.EQUIDISTANT, 672.0, math.pi)):
        lens = oracle64.make_lens(1280, 1024, proj, f, fov, centre=(3.5, -2.25), k=(-1.0e-7, 2.0e-14))
        for _ in range(300):
            v = rng.normal(size=3)
            v[0] = abs(v[0]) + 0.2
            v /= np.linalg.norm(v)
            assert bits_equal(oracle64.fn_project(v, lens), reference64.fn_project(v, lens))
            px = np.array([rng.uniform(0, 1279), rng.uniform(0, 1023)])
            assert bits_equal(oracle64.fn_unproject(px, lens), reference64.fn_unproject(px, lens))
    for act in (wl.SELU, wl.RELU, wl.SOFTMAX, wl.TANH):
        d = rng.normal(0, 2, (50, 7))
        assert bits_equal(oracle64.fn_activation(act, d, 7), reference64.fn_activation(act, d, 7))


# ---- the engine's host-side C++ instantiated with double (Mesh<double, Model>, VisualMesh<double, Model>) ----------
HOST_MESHES = [
    (wl.RING6, wl.SPHERE, 0.0949, 1.2, 6.0, 20.0),
    (wl.RING6, wl.SPHERE, 0.2, 1.0, 1.0, 3.0),
    (wl.RING6, wl.CIRCLE, 0.05, 0.9, 5.0, 4.0),
    (wl.NMGRID8, wl.CIRCLE, 0.05, 1.2, 8.0, 2.0),
    (wl.NMGRID8, wl.SPHERE, 0.0949, 1.0, 4.0, 5.0),
]
HOST_LENSES = [(1280, 1024, wl.EQUISOLID, 420.0, math.pi), (1280, 1024, wl.RECTILINEAR, 700.0, math.pi / 2),
               (2048, 1536, wl.EQUIDISTANT, 672.0, math.pi), (640, 480, wl.RECTILINEAR, 350.0, 1.9)]


@pytest.mark.parametrize("args", HOST_MESHES)
def test_host_mesh_and_lookup_in_double(oracle64, args):
    from visualmesh_amd import engine as eng
    from visualmesh_amd import native
    a, b = eng.Mesh64(*args), oracle64.mesh(*args)
    assert a.n_nodes == b.n_nodes and a.n_neighbours == b.n_neighbours and a.h == b.h
    assert a.arrays()[0].dtype == np.float64
    assert bits_equal(a.arrays()[0], b.arrays()[0]) and bits_equal(a.arrays()[1], b.arrays()[1])
    rng = np.random.default_rng(5)
    for (W, H, proj, f, fov) in HOST_LENSES:
        for i in range(8):
            Hoc = wl.make_hoc(args[3], math.radians(rng.uniform(-30, 110)), math.radians(rng.uniform(-30, 30)),
                              math.radians(rng.uniform(-180, 180)), dtype=np.float64)
            centre = (float(rng.uniform(-20, 20)), float(rng.uniform(-20, 20)))
            k = (0.0, 0.0) if i < 6 else (-1.2e-7, 3.0e-14)
            la = native.make_lens64(W, H, proj, f, fov, centre=centre, k=k)
            lb = oracle64.make_lens(W, H, proj, f, fov, centre=centre, k=k)
            assert bits_equal(a.lookup(Hoc, la), b.lookup(Hoc, lb))


def test_host_visualmesh_in_double(oracle64):
    from visualmesh_amd import engine as eng
    args = (wl.RING6, wl.SPHERE, 0.0949, 0.8, 1.5, 6.0, 0.5, 20.0)
    a, b = eng.VisualMesh64(*args), oracle64.visualmesh(*args)
    assert [m.h for m in a.meshes] == [m.h for m in b.meshes]
    for ma, mb in zip(a.meshes, b.meshes):
        assert bits_equal(ma.arrays()[0], mb.arrays()[0]) and bits_equal(ma.arrays()[1], mb.arrays()[1])
    heights = [m.h for m in a.meshes]
    for h in list(np.linspace(0.6, 1.7, 45)) + heights + [(x + y) / 2 for x, y in zip(heights, heights[1:])]:
        assert a.height(float(h)).h == b.height(float(h)).h


# ---- Engine<double> on the GPU against the oracle in double ---------------------------------------------------------
PX_TOL_F64 = 1e-9     # pixels: the device's acos/sin/tan against glibc's, a few ulp of a coordinate of ~1e3
PROB_TOL_F64 = 1e-9   # absolute; measured ~1e-15 (summation order of the fp64 matrix instruction, exp)


def _assert_parity64(got, want, classify=True, label=""):
    assert got["px"].dtype == np.float64
    assert np.array_equal(got["gidx"], want["gidx"]), label + " global indices differ"
    assert np.array_equal(got["nb"], want["nb"]), label + " neighbourhood differs"
    if len(want["px"]):
        err = np.abs(got["px"] - want["px"]).max()
        assert err <= PX_TOL_F64, "%s pixel coordinates differ by %g px" % (label, err)
    if classify:
        assert got["cls"].shape == want["cls"].shape and got["cls"].dtype == np.float64
        if want["cls"].size:
            err = np.abs(got["cls"] - want["cls"]).max()
            assert err <= PROB_TOL_F64, "%s class probabilities differ by %g" % (label, err)


@pytest.mark.gpu
@pytest.mark.parametrize("index", [1, 3])
def test_gpu_double_engine_on_configurations(oracle64, index):
    """configuration 1 (Ring6, RGBA, equisolid) and 3 (NMGrid8, Bayer, rectilinear) through Engine<double>: indices and
    neighbourhood bit-exact, pixels and probabilities to the gates above"""
    from visualmesh_amd import engine as eng
    from visualmesh_amd import native
    cfg = wl.config(index)
    args = (cfg.model, cfg.shape, cfg.radius, cfg.mesh_h, cfg.k, min(cfg.max_distance, 3.0) if index == 3 else cfg.max_distance)
    om, em = oracle64.mesh(*args), eng.Mesh64(*args)
    groups = network64(cfg.network)
    engine = eng.Engine64(groups, cfg.model)
    f = cfg.frames[0]
    Hoc = f["Hoc"].astype(np.float64)
    want = om.classify(Hoc, oracle64.make_lens(*cfg.lens_tuple()), f["image"], cfg.fourcc, oracle64.network(groups))
    got = engine(em, Hoc, native.make_lens64(*cfg.lens_tuple()), f["image"], cfg.fourcc)
    assert len(want["gidx"]) > 1000
    _assert_parity64(got, want, label="cfg%d" % index)
    proj = engine(em, Hoc, native.make_lens64(*cfg.lens_tuple()))
    _assert_parity64(proj, want, classify=False, label="cfg%d projection" % index)
    # a second call on the same engine gives the same answer (the reference's engine is only right on its first)
    again = engine(em, Hoc, native.make_lens64(*cfg.lens_tuple()), f["image"], cfg.fourcc)
    assert bits_equal(again["cls"], got["cls"]) and bits_equal(again["px"], got["px"])


@pytest.mark.gpu
def test_gpu_double_engine_layer_shapes_and_activations(oracle64):
    """multi-layer groups, every activation, widths that are no multiple of the matrix tile (5, 12, 40, 70), a hidden
    layer wider than one pass of the kernel (136), VisualMesh<double>, three lens models and distortion"""
    from visualmesh_amd import engine as eng
    from visualmesh_amd import native
    rng = np.random.default_rng(21)

    def layer(n_in, n_out, act, scale=0.3):
        return (rng.normal(0, scale / math.sqrt(n_in / 28.0), (n_in, n_out)), rng.normal(0, 0.1, n_out), act)

    groups = [
        [layer(28, 12, wl.TANH), layer(12, 40, wl.RELU)],
        [layer(280, 70, wl.SELU), layer(70, 136, wl.TANH), layer(136, 5, wl.SELU)],
        [layer(35, 3, wl.SOFTMAX)],
    ]
    vargs = (wl.RING6, wl.SPHERE, 0.0949, 0.9, 1.3, 4.0, 0.5, 10.0)
    ov, ev = oracle64.visualmesh(*vargs), eng.VisualMesh64(*vargs)
    engine = eng.Engine64(groups, wl.RING6)
    net = oracle64.network(groups)
    for i, (W, H, proj, f, fov, fcc, bpp) in enumerate([(640, 512, wl.EQUISOLID, 210.0, math.pi, "RGBA", 4),
                                                         (640, 480, wl.RECTILINEAR, 350.0, 1.9, "BGR8", 3),
                                                         (800, 600, wl.EQUIDISTANT, 260.0, math.pi, "GRAY", 1)]):
        k = (0.0, 0.0) if i == 0 else (-1.0e-7, 2.0e-14)
        h = float(rng.uniform(0.9, 1.3))
        Hoc = wl.make_hoc(h, math.radians(rng.uniform(20, 50)), 0.03, -0.02, dtype=np.float64)
        img = wl.random_image(rng, W, H, bpp)
        want = ov.height(h).classify(Hoc, oracle64.make_lens(W, H, proj, f, fov, centre=(2.5, -1.25), k=k), img, wl.fourcc(fcc), net)
        got = engine(ev, Hoc, native.make_lens64(W, H, proj, f, fov, centre=(2.5, -1.25), k=k), img, wl.fourcc(fcc))
        assert len(want["gidx"]) > 100
        _assert_parity64(got, want, label="lens %d" % i)


@pytest.mark.gpu
def test_gpu_double_engine_edges(oracle64):
    """nothing visible, an empty network (the sampled input comes back), an unsupported format, and the edge guard: with
    the device's pixels pushed off by 0.25 px the host must overrule it and the result stays the reference's"""
    from visualmesh_amd import engine as eng
    from visualmesh_amd import native
    args = (wl.RING6, wl.SPHERE, 0.0949, 1.0, 3.0, 8.0)
    om, em = oracle64.mesh(*args), eng.Mesh64(*args)
    lens_o, lens_e = oracle64.make_lens(320, 256, wl.EQUISOLID, 105.0, math.pi), native.make_lens64(320, 256, wl.EQUISOLID, 105.0, math.pi)
    rng = np.random.default_rng(2)
    img = wl.random_image(rng, 320, 256, 4)
    empty = eng.Engine64([], wl.RING6)
    Hoc = wl.make_hoc(1.0, math.radians(35), 0.03, -0.02, dtype=np.float64)
    want = om.classify(Hoc, lens_o, img, wl.fourcc("RGBA"), oracle64.network([]))
    got = empty(em, Hoc, lens_e, img, wl.fourcc("RGBA"))
    assert got["cls"].shape[1] == 4
    _assert_parity64(got, want, label="empty network")
    up = wl.make_hoc(1.0, math.radians(-80), 0.0, 0.0, dtype=np.float64)   # a narrow lens that looks at the sky
    narrow_o, narrow_e = oracle64.make_lens(320, 256, wl.RECTILINEAR, 175.0, 1.9), native.make_lens64(320, 256, wl.RECTILINEAR, 175.0, 1.9)
    assert len(om.project(up, narrow_o)["gidx"]) == 0
    sky = empty(em, up, narrow_e, img, wl.fourcc("RGBA"))
    assert len(sky["gidx"]) == 0 and sky["cls"].size == 0
    assert empty(em, up, narrow_e)["nb"].shape == (1, 6)
    with pytest.raises(ValueError):
        empty(em, Hoc, lens_e, img, wl.fourcc("YUYV"))
    lib = native.hip()
    try:
        native.hip_check(lib.vmhip_debug_set(native.DEBUG_PROJECTION_ERROR, 0.25))
        native.hip_check(lib.vmhip_debug_set(native.DEBUG_EDGE_BAND, 0.5))
        guarded = eng.Engine64([], wl.RING6)
        got = guarded(em, Hoc, lens_e)
        stats = guarded.guard_stats()
    finally:
        native.hip_check(lib.vmhip_debug_set(native.DEBUG_PROJECTION_ERROR, 0.0))
        native.hip_check(lib.vmhip_debug_set(native.DEBUG_EDGE_BAND, 0.0))
    assert np.array_equal(got["gidx"], want["gidx"]) and np.array_equal(got["nb"], want["nb"])
    assert stats["listed"] > 0 and stats["overruled"] > 0
    assert np.abs(got["px"] - want["px"]).max() <= 0.25 + 1e-9

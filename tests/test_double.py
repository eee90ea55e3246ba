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

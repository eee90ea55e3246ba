"""Shared helpers of the parity tests."""
import numpy as np

from oracle import vmo
from visualmesh_amd import engine as eng
from visualmesh_amd import native
from visualmesh_amd import workloads as wl

# parity gates
PX_TOL = 1e-3      # pixels
PROB_TOL = 1e-4    # absolute, fp32 class probabilities
BF16_TOL = 1e-2    # absolute, bf16 variant


def bits_equal(a, b):
    a, b = np.ascontiguousarray(a), np.ascontiguousarray(b)
    if a.shape != b.shape or a.dtype != b.dtype:
        return False
    if a.dtype == np.float32:
        return np.array_equal(a.view(np.uint32), b.view(np.uint32))
    if a.dtype == np.float64:
        return np.array_equal(a.view(np.uint64), b.view(np.uint64))
    return np.array_equal(a, b)


def lens_pair(cfg):
    """(oracle lens, engine lens) of a workload configuration"""
    return vmo.make_lens(*cfg.lens_tuple()), native.make_lens(*cfg.lens_tuple())


def meshes_for(cfg, O):
    """(oracle mesh-or-visualmesh, engine mesh-or-visualmesh)"""
    if cfg.visualmesh is None:
        args = (cfg.model, cfg.shape, cfg.radius, cfg.mesh_h, cfg.k, cfg.max_distance)
        return O.mesh(*args), eng.Mesh(*args)
    v = cfg.visualmesh
    args = (cfg.model, cfg.shape, cfg.radius, v["min_h"], v["max_h"], cfg.k, v["max_error"], cfg.max_distance)
    return O.visualmesh(*args), eng.VisualMesh(*args)


def pick(mesh, Hoc):
    return mesh.height(float(Hoc[2][3])) if hasattr(mesh, "height") else mesh


def assert_projection_parity(got, want, label=""):
    assert len(got["gidx"]) == len(want["gidx"]), "%s visible count %d != %d" % (label, len(got["gidx"]), len(want["gidx"]))
    assert np.array_equal(got["gidx"], want["gidx"]), label + " global indices differ"
    assert np.array_equal(got["nb"], want["nb"]), label + " neighbourhood differs"
    if len(want["px"]):
        err = np.abs(got["px"] - want["px"]).max()
        assert err <= PX_TOL, "%s pixel coordinates differ by %g px" % (label, err)


def assert_classification_parity(got, want, tol=PROB_TOL, label=""):
    assert_projection_parity(got, want, label)
    assert got["cls"].shape == want["cls"].shape, label + " classification shape"
    if want["cls"].size:
        err = np.abs(got["cls"] - want["cls"]).max()
        assert err <= tol, "%s class probabilities differ by %g (gate %g)" % (label, err, tol)

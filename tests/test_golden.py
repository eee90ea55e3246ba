"""The committed golden fixtures (tests/golden/golden.json, written while the compiled reference agreed with
the oracle) against the oracle and against the engine's host-side C++ (mesh generation, BSP lookup). This is
what pins the exact node order and the heuristic lookup ranges on machines without the reference tree."""
import hashlib
import json
import math
import os
import sys

import numpy as np
import pytest

from oracle import vmo
from visualmesh_amd import engine as eng
from visualmesh_amd import native
from visualmesh_amd import workloads as wl

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "golden"))
import make_golden  # noqa: E402

GOLDEN = json.load(open(os.path.join(HERE, "golden", "golden.json")))


def sha(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def test_fixture_was_written_with_the_reference_in_agreement():
    assert GOLDEN["agreed_with_compiled_reference"] is True


@pytest.mark.parametrize("name", sorted(GOLDEN["meshes"]))
def test_oracle_reproduces_golden(oracle, name):
    g = GOLDEN["meshes"][name]
    mesh = oracle.mesh(*make_golden.MESHES[name])
    rays, nbr = mesh.arrays()
    assert mesh.n_nodes == g["n_nodes"]
    assert sha(nbr) == g["neighbours_sha256"]
    assert sha(rays) == g["rays_sha256"], "node rays differ (a different C library can do this; integers must still hold)"
    net = make_golden.network_for(mesh.n_neighbours, 77)
    frames = iter(g["frames"])
    for lname, largs in make_golden.LENSES.items():
        lens = vmo.make_lens(*largs)
        bayer = lname == "rectilinear"
        image = make_golden.image_for(largs, 1 if bayer else 4, 5)
        fcc = wl.fourcc("GRBG") if bayer else wl.fourcc("RGBA")
        for (pitch, roll, yaw) in make_golden.POSES:
            f = next(frames)
            Hoc = wl.make_hoc(make_golden.MESHES[name][3], math.radians(pitch), math.radians(roll), math.radians(yaw))
            r = mesh.classify(Hoc, lens, image, fcc, vmo.Network(net))
            V = len(r["gidx"])
            assert (len(r["ranges"]), V) == (f["n_ranges"], f["visible"])
            assert sha(r["ranges"]) == f["ranges_sha256"] and sha(r["gidx"]) == f["gidx_sha256"] and sha(r["nb"]) == f["nb_sha256"]
            if V:
                rows = np.array(f["sample_rows"])
                assert r["gidx"][rows].tolist() == f["sample_gidx"]
                assert np.abs(r["px"][rows] - np.array(f["sample_px"], np.float32)).max() <= 1e-3
                assert np.abs(r["cls"][rows] - np.array(f["sample_cls"], np.float32)).max() <= 1e-5
                assert np.abs(r["cls"][V] - np.array(f["null_cls"], np.float32)).max() <= 1e-5


@pytest.mark.parametrize("name", sorted(GOLDEN["meshes"]))
def test_host_mesh_code_reproduces_golden(name):
    """visualmesh_amd/cpp: Mesh construction and Mesh::lookup, the host side of the engine."""
    g = GOLDEN["meshes"][name]
    mesh = eng.Mesh(*make_golden.MESHES[name])
    rays, nbr = mesh.arrays()
    assert mesh.n_nodes == g["n_nodes"]
    assert sha(nbr) == g["neighbours_sha256"]
    assert sha(rays) == g["rays_sha256"]
    frames = iter(g["frames"])
    for lname, largs in make_golden.LENSES.items():
        lens = native.make_lens(*largs)
        for (pitch, roll, yaw) in make_golden.POSES:
            f = next(frames)
            Hoc = wl.make_hoc(make_golden.MESHES[name][3], math.radians(pitch), math.radians(roll), math.radians(yaw))
            ranges = mesh.lookup(Hoc, lens)
            assert len(ranges) == f["n_ranges"] and sha(ranges) == f["ranges_sha256"]

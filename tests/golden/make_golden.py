"""Writes tests/golden/golden.json: small fixtures that pin the host-side mesh code, the lookup ranges and
the engine's outputs on machines where the reference tree is not mounted.

Run from the repository root:  python tests/golden/make_golden.py
The values come from the CPU oracle; when the compiled reference (oracle/_ref/libvm_ref.so) is present the
script refuses to write unless the reference produces exactly the same values, so a committed fixture is
one the reference agreed with. Integer data is stored as SHA-256 digests plus a few verbatim entries; floats
as verbatim samples (compared with a tolerance, the C library may differ between machines).
"""
import hashlib
import json
import math
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)

from oracle import vmo  # noqa: E402
from visualmesh_amd import workloads as wl  # noqa: E402

MESHES = {
    "ring6_sphere_k6": (wl.RING6, wl.SPHERE, 0.0949, 1.2, 6.0, 20.0),
    "ring6_sphere_k4_h08": (wl.RING6, wl.SPHERE, 0.0949, 0.8, 4.0, 10.0),
    "ring6_circle_k5": (wl.RING6, wl.CIRCLE, 0.05, 0.9, 5.0, 4.0),
    "nmgrid8_circle_k8": (wl.NMGRID8, wl.CIRCLE, 0.05, 1.2, 8.0, 2.0),
    "nmgrid8_sphere_k4": (wl.NMGRID8, wl.SPHERE, 0.0949, 1.0, 4.0, 5.0),
}
LENSES = {
    "equisolid": (1280, 1024, wl.EQUISOLID, 420.0, math.pi),
    "rectilinear": (1280, 1024, wl.RECTILINEAR, 700.0, math.pi / 2),
    "equidistant": (2048, 1536, wl.EQUIDISTANT, 672.0, math.pi),
}
POSES = [(30.0, 3.0, -2.0), (10.0, -5.0, 120.0), (60.0, 0.0, 0.0), (85.0, 4.0, -170.0), (-40.0, 0.0, 10.0)]


def sha(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def network_for(nn, seed):
    rng = np.random.default_rng(seed)
    return wl.glorot_network(rng, [3, 8, 8, 3], nn, wl.SELU if nn == 6 else wl.RELU)


def image_for(lens, bpp, seed):
    return wl.random_image(np.random.default_rng(seed), lens[0], lens[1], bpp)


def build(O):
    out = {"glibc": os.confstr("CS_GNU_LIBC_VERSION"), "meshes": {}}
    for mname, margs in MESHES.items():
        mesh = O.mesh(*margs)
        rays, nbr = mesh.arrays()
        entry = {"args": list(margs), "n_nodes": mesh.n_nodes, "rays_sha256": sha(rays), "neighbours_sha256": sha(nbr),
                 "first_rays": rays[:4].tolist(), "first_neighbours": nbr[:4].tolist(), "frames": []}
        nn = mesh.n_neighbours
        net = network_for(nn, 77)
        for lname, largs in LENSES.items():
            lens = vmo.make_lens(*largs)
            bayer = lname == "rectilinear"
            image = image_for(largs, 1 if bayer else 4, 5)
            fcc = wl.fourcc("GRBG") if bayer else wl.fourcc("RGBA")
            for pi, (pitch, roll, yaw) in enumerate(POSES):
                Hoc = wl.make_hoc(margs[3], math.radians(pitch), math.radians(roll), math.radians(yaw))
                r = mesh.classify(Hoc, lens, image, fcc, vmo.Network(net))
                V = len(r["gidx"])
                pick = np.linspace(0, V - 1, 8).astype(int) if V else np.zeros(0, int)
                entry["frames"].append({
                    "lens": lname, "pose": [pitch, roll, yaw], "n_ranges": int(len(r["ranges"])), "ranges_sha256": sha(r["ranges"]),
                    "visible": V, "gidx_sha256": sha(r["gidx"]), "nb_sha256": sha(r["nb"]),
                    "sample_rows": pick.tolist(), "sample_gidx": r["gidx"][pick].tolist() if V else [],
                    "sample_px": r["px"][pick].tolist() if V else [], "sample_cls": r["cls"][pick].tolist() if V else [],
                    "null_cls": r["cls"][V].tolist() if V else [],
                })
        out["meshes"][mname] = entry
    return out


if __name__ == "__main__":
    data = build(vmo.load("oracle"))
    ref = vmo.load("reference")
    if ref is not None:
        want = build(ref)
        assert json.dumps(want, sort_keys=True) == json.dumps(data, sort_keys=True), "oracle and reference disagree"
        data["agreed_with_compiled_reference"] = True
    else:
        data["agreed_with_compiled_reference"] = False
    with open(os.path.join(HERE, "golden.json"), "w") as f:
        json.dump(data, f, indent=1, sort_keys=True)
    print("wrote golden.json; reference agreed:", data["agreed_with_compiled_reference"])

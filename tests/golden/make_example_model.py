"""Writes tests/golden/example_model.npz and tests/golden/example_poses.json: the weights of the reference's
exported example network (example/model.yaml, 13 graph-convolution layers, 5 classes) and the lens and camera pose of
its 30 dataset elements (example/images/lens*.yaml, with the size of the image next to each), as plain data, so that
the network and the poses can be used on machines where the reference tree is not mounted.

Run from the repository root:  python tests/golden/make_example_model.py
The files are read with the repository's own C++ reader (visualmesh/utility/load_model.hpp) and the script refuses to
write unless PyYAML reads the same values.
"""
import glob
import json
import os
import sys

import numpy as np
import yaml
from PIL import Image

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)

from visualmesh_amd import engine as eng  # noqa: E402

EXAMPLE = "/root/reference/example"


def main():
    model = eng.load_model(os.path.join(EXAMPLE, "model.yaml"))
    check = yaml.safe_load(open(os.path.join(EXAMPLE, "model.yaml")))
    arrays = {}
    activations = []
    for g, (group, ref_group) in enumerate(zip(model["network"], check["network"])):
        assert len(group) == len(ref_group)
        for l, ((w, b, act), ref_layer) in enumerate(zip(group, ref_group)):
            assert np.array_equal(w, np.array(ref_layer["weights"], np.float32)), (g, l)
            assert np.array_equal(b, np.array(ref_layer["biases"], np.float32)), (g, l)
            arrays["w_%d_%d" % (g, l)] = w
            arrays["b_%d_%d" % (g, l)] = b
            activations.append([g, l, int(act)])
    arrays["activations"] = np.array(activations, np.int32)
    np.savez_compressed(os.path.join(HERE, "example_model.npz"), **arrays)

    poses = []
    for path in sorted(glob.glob(os.path.join(EXAMPLE, "images", "lens*.yaml"))):
        number = os.path.basename(path)[4:11]
        width, height = Image.open(os.path.join(EXAMPLE, "images", "image%s.jpg" % number)).size
        lens, Hoc = eng.load_lens(path, width, height)
        ref = yaml.safe_load(open(path))
        assert np.array_equal(Hoc, np.array(ref["Hoc"], np.float32)), path
        assert abs(lens.focal_length - ref["focal_length"]) < 1e-3 and lens.fov == np.float32(ref["fov"]), path
        poses.append(dict(number=number, width=width, height=height, projection=ref["projection"],
                          focal_length=float(lens.focal_length), centre=[float(lens.centre[0]), float(lens.centre[1])],
                          k=[float(lens.k[0]), float(lens.k[1])], fov=float(lens.fov), Hoc=[[float(v) for v in row] for row in Hoc]))
    meta = dict(mesh=model["mesh"], shape=model["shape"], radius=float(model["radius"]), intersections=float(model["intersections"]),
                poses=poses)
    with open(os.path.join(HERE, "example_poses.json"), "w") as f:
        json.dump(meta, f, indent=1)
    print("wrote %d layers and %d poses" % (len(activations), len(poses)))


if __name__ == "__main__":
    main()

"""The C++ reader for exported models and dataset lens files (visualmesh/utility/load_model.hpp on yaml_lite.hpp):
against PyYAML on the reference's own example files where the reference tree is mounted, against the committed
fixtures made from them, and on hand-written documents that use the YAML forms the reader claims to support."""
import json
import os

import numpy as np
import pytest

from visualmesh_amd import engine as eng

HERE = os.path.dirname(os.path.abspath(__file__))
EXAMPLE = "/root/reference/example"
needs_reference = pytest.mark.skipif(not os.path.isdir(EXAMPLE), reason="the reference tree is not mounted")


@needs_reference
def test_example_model_matches_pyyaml():
    import yaml
    got = eng.load_model(os.path.join(EXAMPLE, "model.yaml"))
    want = yaml.safe_load(open(os.path.join(EXAMPLE, "model.yaml")))
    assert got["mesh"] == want["mesh"] and got["shape"] == want["geometry"]["shape"]
    assert got["radius"] == np.float32(want["geometry"]["radius"])
    assert len(got["network"]) == len(want["network"]) == 13
    names = {0: "selu", 1: "relu", 2: "softmax", 3: "tanh"}
    for group, ref_group in zip(got["network"], want["network"]):
        assert len(group) == len(ref_group)
        for (w, b, act), ref in zip(group, ref_group):
            assert np.array_equal(w, np.array(ref["weights"], np.float32))
            assert np.array_equal(b, np.array(ref["biases"], np.float32))
            assert names[act] == ref["activation"]


@needs_reference
def test_example_lens_files_match_pyyaml():
    import yaml
    for i in (0, 7, 29):
        path = os.path.join(EXAMPLE, "images", "lens%07d.yaml" % i)
        lens, Hoc = eng.load_lens(path, 1280, 1024)
        want = yaml.safe_load(open(path))
        assert np.array_equal(Hoc, np.array(want["Hoc"], np.float32))
        assert lens.focal_length == np.float32(want["focal_length"]) and lens.fov == np.float32(want["fov"])
        assert (lens.width, lens.height) == (1280, 1024)
        assert {"RECTILINEAR": 0, "EQUISOLID": 1, "EQUIDISTANT": 2}[want["projection"]] == lens.projection
        assert [lens.centre[0], lens.centre[1], lens.k[0], lens.k[1]] == [np.float32(v) for v in want["centre"] + want["k"]]


@needs_reference
def test_fixtures_are_the_example_files():
    got = eng.load_model(os.path.join(EXAMPLE, "model.yaml"))
    fixture = np.load(os.path.join(HERE, "golden", "example_model.npz"))
    for g, l, act in fixture["activations"]:
        w, b, a = got["network"][g][l]
        assert np.array_equal(w, fixture["w_%d_%d" % (g, l)]) and np.array_equal(b, fixture["b_%d_%d" % (g, l)]) and a == act
    poses = json.load(open(os.path.join(HERE, "golden", "example_poses.json")))["poses"]
    assert len(poses) == 30
    lens, Hoc = eng.load_lens(os.path.join(EXAMPLE, "images", "lens%s.yaml" % poses[3]["number"]), poses[3]["width"], poses[3]["height"])
    assert np.array_equal(Hoc, np.array(poses[3]["Hoc"], np.float32))


DOCUMENT = """\
# an exported model, written by hand with every form the reader supports
geometry: { shape: "SPHERE", radius: 0.1, intersections: 6 }   # flow mapping, quoted scalar
mesh: 'RING6'
network:
  - - activation: selu          # sequence of sequences of mappings, nested on one line
      biases: [0.5, -1.5e-1]
      weights:
        - [1, 2]
        - [3.5,
           -4.25]               # a flow sequence that continues on the next line
      ignored: ~
  -
    - weights:                   # the item starts on the next line; sequence at the key's own indentation
      - [0.25]
      - [-.5]
      activation: "softmax"
      biases: [1.0e+0]
"""


def test_yaml_forms(tmp_path):
    path = tmp_path / "model.yaml"
    path.write_text(DOCUMENT)
    m = eng.load_model(path)
    assert (m["mesh"], m["shape"]) == ("RING6", "SPHERE")
    assert m["radius"] == np.float32(0.1) and m["intersections"] == 6.0
    assert len(m["network"]) == 2 and len(m["network"][0]) == 1 and len(m["network"][1]) == 1
    w, b, act = m["network"][0][0]
    assert act == 0 and np.array_equal(w, np.array([[1, 2], [3.5, -4.25]], np.float32)) and np.array_equal(b, np.array([0.5, -0.15], np.float32))
    w, b, act = m["network"][1][0]
    assert act == 2 and np.array_equal(w, np.array([[0.25], [-0.5]], np.float32)) and np.array_equal(b, np.array([1.0], np.float32))


@pytest.mark.parametrize("text, message", [
    ("network:\n  - - activation: swish\n      biases: [0]\n      weights:\n        - [1]\n", "Unknown activation function swish"),
    ("network:\n  - - activation: selu\n      biases: [0, 1]\n      weights:\n        - [1]\n", "does not match"),
    ("network:\n  - - activation: selu\n      biases: [zero]\n      weights:\n        - [1]\n", "not a number"),
    ("network:\n  - - activation: selu\n      biases: [0\n", "unterminated"),
    ("mesh: RING6\n", "key 'network' not found"),
    ("network: &anchor\n  - []\n", "not supported"),
])
def test_malformed_models_are_reported(tmp_path, text, message):
    path = tmp_path / "bad.yaml"
    path.write_text(text)
    with pytest.raises(RuntimeError) as err:
        eng.load_model(path)
    assert message in str(err.value)


def test_missing_file_is_reported(tmp_path):
    with pytest.raises(RuntimeError) as err:
        eng.load_model(tmp_path / "nothing.yaml")
    assert "cannot open" in str(err.value)

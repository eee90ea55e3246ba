"""HIP engine against the CPU oracle on the benchmark configurations, through the C++ engine and so
through the C ABI. Gates: visible-node indices and neighbour tables bit-exact, pixel coordinates within
1e-3 px, fp32 class probabilities within 1e-4 absolute."""
import math

import numpy as np
import pytest

from helpers import (BF16_TOL, PROB_TOL, assert_classification_parity, assert_projection_parity, lens_pair, meshes_for, pick)
from oracle import vmo
from visualmesh_amd import engine as eng
from visualmesh_amd import native
from visualmesh_amd import workloads as wl

pytestmark = pytest.mark.gpu


def _run_config(oracle, index, n_frames, batch, check_cls_frames=None):
    cfg = wl.config(index, n_frames=n_frames)
    o_lens, e_lens = lens_pair(cfg)
    o_mesh, e_mesh = meshes_for(cfg, oracle)
    engine = eng.Engine(cfg.network, cfg.model)
    net = vmo.Network(cfg.network)
    if batch:
        frames = [dict(mesh=e_mesh, Hoc=f["Hoc"], lens=e_lens, image=f["image"], fourcc=cfg.fourcc) for f in cfg.frames]
        results = engine.classify_batch(frames)
    else:
        results = [engine(e_mesh, f["Hoc"], e_lens, f["image"], cfg.fourcc) for f in cfg.frames]
    for i, f in enumerate(cfg.frames):
        label = "%s frame %d" % (cfg.name, i)
        print(label, "V =", len(results[i]["gidx"]), flush=True)
        if check_cls_frames is None or i in check_cls_frames:
            want = pick(o_mesh, f["Hoc"]).classify(f["Hoc"], o_lens, f["image"], cfg.fourcc, net)
            assert_classification_parity(results[i], want, PROB_TOL, label)
            # the null row is an ordinary row
            assert results[i]["cls"].shape[0] == len(results[i]["gidx"]) + 1
        else:
            want = pick(o_mesh, f["Hoc"]).project(f["Hoc"], o_lens)
            assert_projection_parity(results[i], want, label)


def test_config1_single_frame(oracle):
    _run_config(oracle, 1, 1, batch=False)


def test_config1_projection_only(oracle):
    cfg = wl.config(1)
    o_lens, e_lens = lens_pair(cfg)
    o_mesh, e_mesh = meshes_for(cfg, oracle)
    engine = eng.Engine([], cfg.model)
    got = engine(e_mesh, cfg.frames[0]["Hoc"], e_lens)
    want = o_mesh.project(cfg.frames[0]["Hoc"], o_lens)
    assert_projection_parity(got, want, "cfg1 projection")


def test_config2_batch(oracle):
    """all 16 frames of the batch against the oracle"""
    _run_config(oracle, 2, 16, batch=True)


def test_config3_bayer(oracle):
    _run_config(oracle, 3, 1, batch=False)


def test_device_libm_matches_host(oracle):
    """The device's acosf/sinf/tanf/sqrtf must return the host C library's bits (a dense sample here; the
    same source is compared exhaustively on the CPU in test_libm_exact.py). The square root is the compiler's
    sequence on the device and not the header's own arithmetic, so it is compared exhaustively here."""
    import ctypes as C
    from visualmesh_amd import native
    L = native.hip()
    rng = np.random.default_rng(7)
    n = 1 << 22
    cases = {
        "acos": (0, np.concatenate([rng.uniform(-1, 1, n).astype(np.float32), (1 - np.geomspace(1e-8, 1, 4096)).astype(np.float32),
                                    np.array([1.0, -1.0, 0.0, 0.5, -0.5], np.float32)])),
        "sin": (1, np.concatenate([rng.uniform(0, np.pi / 2, n).astype(np.float32), np.geomspace(1e-7, 1.6, 4096).astype(np.float32)])),
        "tan": (2, np.concatenate([rng.uniform(0, np.pi / 2, n).astype(np.float32), (np.float32(np.pi / 2) - np.geomspace(1e-7, 1, 4096)).astype(np.float32),
                                   np.array([np.float32(np.pi / 2)], np.float32)])),
    }

    def all_cases():
        for name, (which, x) in cases.items():
            yield name, which, x
        # the square root over every float from zero to four, denormals included (the projection takes roots of values in [0, 1])
        step = 1 << 26
        for first in range(0, 0x40800000 + 1, step):
            yield "sqrt from bit pattern %#x" % first, 3, np.arange(first, min(first + step, 0x40800000 + 1), dtype=np.uint32).view(np.float32)

    for name, which, x in all_cases():
        x = np.ascontiguousarray(x)
        y = np.zeros_like(x)
        native.hip_check(L.vmhip_selftest_libm(which, x.ctypes.data_as(C.POINTER(C.c_float)), y.ctypes.data_as(C.POINTER(C.c_float)), x.size))
        want = oracle.fn_libm(name.split()[0], x)
        bad = np.flatnonzero(y.view(np.uint32) != want.view(np.uint32))
        assert bad.size == 0, "%s: %d of %d differ, e.g. x=%r device=%r host=%r" % (name, bad.size, x.size, x[bad[0]], y[bad[0]], want[bad[0]])


@pytest.mark.parametrize("row_bits,runs", [(0, 600), (30, 40), (31, 12)], ids=["8-bit stamp", "2-bit stamp", "1-bit stamp"])
def test_reverse_lookup_across_a_restart_of_the_run_stamp(oracle, row_bits, runs):
    """A reverse-lookup entry holds an 8-bit run stamp above the row, and an engine's table is cleared when the stamps
    start again after 255 runs. One view stamps its nodes, then two other views take turns 600 times on the same engine:
    no run may take an entry of the first view (or of a run 255 runs earlier) for current. A frame of 2^24 candidates
    or more leaves fewer bits for the stamp; the knob makes ordinary frames do so (stamps start again every 3 runs, and
    every run)."""
    lib = native.hip()
    native.hip_check(lib.vmhip_debug_set(native.DEBUG_STAMP_ROW_BITS, row_bits))
    try:
        _stamp_restart(oracle, runs)
    finally:
        native.hip_check(lib.vmhip_debug_set(native.DEBUG_STAMP_ROW_BITS, 0))


def _stamp_restart(oracle, runs):
    mesh = eng.Mesh(wl.RING6, wl.SPHERE, 0.0949, 1.0, 3.0, 8.0)
    lens = native.make_lens(320, 256, wl.RECTILINEAR, 180.0, math.pi / 2)
    first_view = wl.make_hoc(1.0, math.radians(50.0), math.radians(-4.0), math.radians(1.0))
    views = [wl.make_hoc(1.0, math.radians(55.0), math.radians(3.0), math.radians(40.0)),
             wl.make_hoc(1.0, math.radians(42.0), math.radians(-2.0), math.radians(65.0))]
    engine = eng.Engine([], wl.RING6)
    a = engine.project(mesh, first_view, lens)
    assert len(a["gidx"]) > 100
    o_mesh = oracle.mesh(wl.RING6, wl.SPHERE, 0.0949, 1.0, 3.0, 8.0)
    o_lens = vmo.make_lens(320, 256, wl.RECTILINEAR, 180.0, math.pi / 2)
    want = []
    for Hoc in views:
        o = o_mesh.project(Hoc, o_lens)
        assert 100 < len(o["gidx"]) and not set(o["gidx"]) >= set(a["gidx"])  # the first view has nodes of its own
        want.append(o)
    for run in range(runs):
        got = engine.project(mesh, views[run & 1], lens)
        assert np.array_equal(got["gidx"], want[run & 1]["gidx"]), "run %d: visible nodes differ" % run
        assert np.array_equal(got["nb"], want[run & 1]["nb"]), "run %d: neighbourhood differs" % run


def test_neighbourhood_of_meshes_with_other_neighbour_counts(oracle):
    """The neighbourhood kernel has instantiations for 4, 6 and 8 neighbours per node and a general one. Meshes with 5
    and with 12 columns of neighbours (the nodes of a real mesh, so that the lookup is a real one; the columns random,
    "no neighbour" included) go through vmhip_project, and the table must be what engine/cpu/engine.hpp:127-143 defines:
    the row of every neighbour that is on screen, the null row for the others."""
    import ctypes as C
    L = native.hip()
    rng = np.random.default_rng(12)
    mesh = eng.Mesh(wl.RING6, wl.SPHERE, 0.0949, 1.0, 3.0, 8.0)
    rays, _ = mesh.arrays()
    lens = native.make_lens(320, 256, wl.EQUISOLID, 105.0, math.pi)
    Hoc = np.ascontiguousarray(wl.make_hoc(1.0, math.radians(40.0), 0.02, 0.3), dtype=np.float32)
    ranges = np.ascontiguousarray(mesh.lookup(Hoc, lens), dtype=np.int32)
    n_cand = int((ranges[:, 1] - ranges[:, 0]).sum())
    Rco = np.ascontiguousarray(Hoc[:3, :3].T)
    empty = native.Network([])
    for nn in (5, 12, 4):
        nbr = np.ascontiguousarray(rng.integers(0, mesh.n_nodes + 1, (mesh.n_nodes, nn)), dtype=np.int32)
        engine, handle = C.c_void_p(), C.c_void_p()
        native.hip_check(L.vmhip_engine_create(C.byref(empty.c), nn, native.FP32, C.byref(engine)))
        native.hip_check(L.vmhip_mesh_upload(rays.ctypes.data_as(C.POINTER(C.c_float)), nbr.ctypes.data_as(C.POINTER(C.c_int32)), mesh.n_nodes, nn, C.byref(handle)))
        px = np.zeros((n_cand, 2), np.float32)
        gidx = np.zeros(n_cand, np.int32)
        nb = np.full((n_cand + 1, nn), -1, np.int32)
        frame = native.Frame(handle, (C.c_float * 9)(*Rco.ravel()), lens, ranges.ctypes.data_as(C.POINTER(C.c_int32)), len(ranges), None, 0, None)
        result = native.Result(n_cand, 0, px.ctypes.data_as(C.POINTER(C.c_float)), gidx.ctypes.data_as(C.POINTER(C.c_int32)),
                               nb.ctypes.data_as(C.POINTER(C.c_int32)), None)
        for _ in range(2):  # the second run finds the first run's stamps in the table
            native.hip_check(L.vmhip_project(engine, C.byref(frame), C.byref(result)))
        V = result.n_visible
        assert V > 500
        row_of = np.full(mesh.n_nodes + 1, V, np.int32)
        row_of[gidx[:V]] = np.arange(V, dtype=np.int32)
        want = np.concatenate([row_of[nbr[gidx[:V]]], np.full((1, nn), V, np.int32)])
        assert np.array_equal(nb[:V + 1], want), "%d neighbours per node" % nn
        L.vmhip_mesh_release(handle)
        L.vmhip_engine_destroy(engine)


def test_neighbourhood_kernel_with_64_bit_offsets(oracle):
    """A batch with a table of 4 GiB or more takes the instantiations of the neighbourhood kernel that address with
    64-bit offsets; the knob forces them onto ordinary frames: projection only (no tile-local tables), a network with
    six neighbours per node, and a batch whose frames differ in their neighbour count (the general instantiation)."""
    lib = native.hip()
    native.hip_check(lib.vmhip_debug_set(native.DEBUG_WIDE_OFFSETS, 1))
    try:
        test_config1_projection_only(oracle)
        _run_config(oracle, 1, 1, batch=False)
        test_neighbourhood_of_meshes_with_other_neighbour_counts(oracle)
    finally:
        native.hip_check(lib.vmhip_debug_set(native.DEBUG_WIDE_OFFSETS, 0))


def test_pixels_and_inputs_bit_exact(oracle):
    """Beyond the 1e-3 px gate: with the host-exact libm the pixel coordinates, and with them the sampled
    network inputs, are bit-identical to the CPU engine's (empty network -> classifications = sampled input)."""
    for index in (1, 3, 4):
        cfg = wl.config(index, n_frames=1)
        o_lens, e_lens = lens_pair(cfg)
        o_mesh, e_mesh = meshes_for(cfg, oracle)
        engine = eng.Engine([], cfg.model)
        f = cfg.frames[0]
        got = engine(e_mesh, f["Hoc"], e_lens, f["image"], cfg.fourcc)
        want = pick(o_mesh, f["Hoc"]).classify(f["Hoc"], o_lens, f["image"], cfg.fourcc, vmo.Network([]))
        assert np.array_equal(got["gidx"], want["gidx"])
        assert np.array_equal(got["px"].view(np.uint32), want["px"].view(np.uint32)), "%s pixel bits" % cfg.name
        assert np.array_equal(got["cls"].view(np.uint32), want["cls"].view(np.uint32)), "%s sampled input bits" % cfg.name


def test_config4_geometry_projection(oracle):
    """Configuration 4's mesh (849k nodes), lens and image size: indices, neighbourhood and pixels on three of
    its random poses (the 64-wide network on this geometry costs the oracle ~45 s per frame, so the
    probabilities are checked on the smaller geometry below)."""
    cfg = wl.config(4, n_frames=3)
    o_lens, e_lens = lens_pair(cfg)
    o_mesh, e_mesh = meshes_for(cfg, oracle)
    engine = eng.Engine([], cfg.model)
    for i, f in enumerate(cfg.frames):
        got = engine(e_mesh, f["Hoc"], e_lens)
        want = o_mesh.project(f["Hoc"], o_lens)
        print("cfg4 frame", i, "V =", len(want["gidx"]), flush=True)
        assert_projection_parity(got, want, "cfg4 frame %d" % i)


def test_config4_network_on_config1_geometry(oracle):
    """The 6 x 64-wide network of configuration 4 (matrix-core kernels, 64-wide softmax) on configuration 1's
    geometry, two frames in one batch."""
    cfg = wl.config(1, n_frames=2)
    net = wl.config(4, n_frames=1).network
    o_lens, e_lens = lens_pair(cfg)
    o_mesh, e_mesh = meshes_for(cfg, oracle)
    engine = eng.Engine(net, cfg.model)
    frames = [dict(mesh=e_mesh, Hoc=f["Hoc"], lens=e_lens, image=f["image"], fourcc=cfg.fourcc) for f in cfg.frames]
    results = engine.classify_batch(frames)
    for i, f in enumerate(cfg.frames):
        want = o_mesh.classify(f["Hoc"], o_lens, f["image"], cfg.fourcc, vmo.Network(net))
        assert_classification_parity(results[i], want, PROB_TOL, "64-wide frame %d" % i)


def test_config4_and_5_full_size_frame(oracle):
    """One frame of configurations 4 and 5 at their real size (2048x1536, ~4.5e5 visible nodes, 6 x 64 network):
    the fp32 engine within 1e-4, the bf16 engine within 1e-2 and the split engine (pairs of bf16 on the bf16 matrix
    instructions) within fp32's 1e-4 of the same oracle result (~45 s of CPU)."""
    cfg = wl.config(4, n_frames=1)
    o_lens, e_lens = lens_pair(cfg)
    o_mesh, e_mesh = meshes_for(cfg, oracle)
    f = cfg.frames[0]
    print("cfg4/5 full-size frame: oracle running", flush=True)
    want = o_mesh.classify(f["Hoc"], o_lens, f["image"], cfg.fourcc, vmo.Network(cfg.network))
    print("cfg4/5 full-size frame: V =", len(want["gidx"]), flush=True)
    for precision, tol, label in ((native.FP32, PROB_TOL, "cfg4 fp32"), (native.BF16, BF16_TOL, "cfg5 bf16"), (native.SPLIT, PROB_TOL, "cfg6 split")):
        engine = eng.Engine(cfg.network, cfg.model, precision=precision)
        got = engine(e_mesh, f["Hoc"], e_lens, f["image"], cfg.fourcc)
        print(label, "worst absolute probability error: %.3e" % float(np.abs(got["cls"] - want["cls"]).max()), flush=True)
        assert_classification_parity(got, want, tol, label)


@pytest.mark.parametrize("index", [1, 3])
def test_layer_shapes_outside_the_enumerated_ones(oracle, index):
    """A network whose widths no kernel was written for, 4 -> 48 -> 40 -> 12 -> 5, on configuration 1's Ring6 and
    configuration 3's NMGrid8 geometry: every layer still runs on a matrix-core kernel (the instantiations that read
    the number of output channels at run time: conv_lds for input rows up to 32 channels, conv_mfma above), within
    1e-4 of the oracle (reference engine/opencl/operation/make_network.hpp:43-214 generates a kernel for any shape)."""
    cfg = wl.config(index, n_frames=1)
    nn = wl.N_NEIGHBOURS[cfg.model]
    rng = np.random.default_rng(123)
    net = wl.glorot_network(rng, [3, 48, 40, 12, 5], nn, wl.SELU if index == 1 else wl.RELU)
    o_lens, e_lens = lens_pair(cfg)
    o_mesh, e_mesh = meshes_for(cfg, oracle)
    engine = eng.Engine(net, cfg.model)
    f = cfg.frames[0]
    got = engine(e_mesh, f["Hoc"], e_lens, f["image"], cfg.fourcc)
    engine.profile(True)
    engine.run()
    names = [n for n, _, _ in engine.profile_read() if n.startswith("conv")]
    s = nn + 1
    assert names == ["conv_lds_4x48s%d" % s, "conv_mfma_48x40s%d" % s, "conv_mfma_40x12s%d" % s, "conv_lds_12x5s%d" % s], names
    want = pick(o_mesh, f["Hoc"]).classify(f["Hoc"], o_lens, f["image"], cfg.fourcc, vmo.Network(net))
    assert got["cls"].shape[1] == 5
    assert_classification_parity(got, want, PROB_TOL, "4->48->40->12->5 on cfg%d" % index)


def test_class_layers_use_the_4x4_matrix_instruction(oracle):
    """The output layers of configurations 1 to 3 (16 -> 2, 16 -> 3, 24 -> 4) run on the kernel built on
    v_mfma_f32_4x4x1 by default; their probabilities are covered by the configuration tests above, this one pins
    the kernel choice those tests exercised."""
    for index, last in ((1, "conv_narrow_16x2s7"), (2, "conv_narrow_16x3s7"), (3, "conv_narrow_24x4s9")):
        cfg = wl.config(index, n_frames=1)
        _, e_lens = lens_pair(cfg)
        _, e_mesh = meshes_for(cfg, oracle)
        engine = eng.Engine(cfg.network, cfg.model)
        f = cfg.frames[0]
        engine(e_mesh, f["Hoc"], e_lens, f["image"], cfg.fourcc)
        frames = [dict(mesh=e_mesh, Hoc=f["Hoc"], lens=e_lens, image=f["image"], fourcc=cfg.fourcc)]
        engine.stage(frames)
        engine.profile(True)
        engine.run()
        names = [n for n, _, _ in engine.profile_read() if n.startswith("conv")]
        assert names[-1] == last, names


def test_bf16_engine(oracle):
    """The bf16 engine (configuration 5's precision and 6 x 64 network) against the fp32 oracle on configuration
    1's geometry: geometry bit-exact, probabilities within 1e-2. The kernel names prove that the bf16
    matrix-instruction kernels were the ones that ran, the error that bf16 rows were really stored."""
    cfg = wl.config(1, n_frames=2)
    net = wl.config(5, n_frames=1).network
    o_lens, e_lens = lens_pair(cfg)
    o_mesh, e_mesh = meshes_for(cfg, oracle)
    engine = eng.Engine(net, cfg.model, precision=native.BF16)
    frames = [dict(mesh=e_mesh, Hoc=f["Hoc"], lens=e_lens, image=f["image"], fourcc=cfg.fourcc) for f in cfg.frames]
    results = engine.classify_batch(frames)
    engine.profile(True)
    engine.run()
    names = [n for n, _, _ in engine.profile_read() if n.startswith("conv")]
    assert names == ["conv_lds_tox2_4x64s7", "conv_bf16_x2_tobf16_64x64s7", "conv_bf16_bf16_tox2_64x64s7", "conv_bf16_x2_tobf16_64x64s7",
                     "conv_bf16_bf16_tox2_64x64s7", "conv_bf16_x2_tof32_64x64s7"], names
    worst = 0.0
    for i, f in enumerate(cfg.frames):
        want = o_mesh.classify(f["Hoc"], o_lens, f["image"], cfg.fourcc, vmo.Network(net))
        assert_classification_parity(results[i], want, BF16_TOL, "bf16 frame %d" % i)
        worst = max(worst, float(np.abs(results[i]["cls"] - want["cls"]).max()))
    print("bf16 worst absolute probability error: %.3e" % worst, flush=True)
    assert worst > PROB_TOL  # two boundaries are stored as bf16: an error this small would mean they were not


@pytest.mark.parametrize("hidden", [3, 10])
def test_bf16_engine_on_other_depths(oracle, hidden):
    """The plan for the rows between bf16 layers - at most two boundaries rounded to bf16, every second one, the others
    hi + lo pairs - was tuned on configuration 5's six layers. What a rounding costs grows with the depth of the network
    (a single one, anywhere, already 0.8-1.5e-2 with ten 64-wide layers), so networks with more than five bf16 layers get
    no rounded boundary. A shallower (three 64-wide layers) and a deeper (ten) network on configuration 1's geometry must
    stay inside the same 1e-2 gate."""
    cfg = wl.config(1, n_frames=1)
    rng = np.random.default_rng(500 + hidden)
    net = wl.glorot_network(rng, [3] + [64] * hidden + [4], 6, wl.SELU)
    o_lens, e_lens = lens_pair(cfg)
    o_mesh, e_mesh = meshes_for(cfg, oracle)
    engine = eng.Engine(net, cfg.model, precision=native.BF16)
    f = cfg.frames[0]
    got = engine(e_mesh, f["Hoc"], e_lens, f["image"], cfg.fourcc)
    engine.stage([dict(mesh=e_mesh, Hoc=f["Hoc"], lens=e_lens, image=f["image"], fourcc=cfg.fourcc)])
    engine.profile(True)
    engine.run()
    names = [n for n, _, _ in engine.profile_read() if n.startswith("conv")]
    assert len(names) == hidden + 1 and all(n.startswith("conv_bf16_") for n in names[1:hidden]), names
    rounded = sum("_tobf16_" in n for n in names)
    assert rounded == (1 if hidden == 3 else 0), names
    want = o_mesh.classify(f["Hoc"], o_lens, f["image"], cfg.fourcc, vmo.Network(net))
    worst = float(np.abs(got["cls"] - want["cls"]).max())
    print("bf16, %d hidden layers: %d boundaries as bf16, worst absolute probability error %.3e" % (hidden, rounded, worst), flush=True)
    assert_classification_parity(got, want, BF16_TOL if rounded else 1e-3, "bf16, %d hidden layers" % hidden)


@pytest.mark.parametrize("hidden", [3, 6, 10])
def test_split_engine_keeps_the_fp32_bar(oracle, hidden):
    """Precision SPLIT: the 64-wide layers on the bf16 matrix instructions with every row between them as pairs of bf16
    and three products per pair of values. Networks of three and six 64-wide layers on configuration 1's geometry must
    stay within the fp32 engine's gate, 1e-4 on the probabilities, and no boundary may be rounded to bf16. What the
    pairs leave out (the product of the two low parts, and a value's bits beyond the sixteenth) adds up with depth:
    1.1e-5, 3.4e-5 and 9.7e-5 at three, six and ten layers, so the ten-layer network is held to 2e-4."""
    cfg = wl.config(1, n_frames=1)
    rng = np.random.default_rng(500 + hidden)
    net = wl.glorot_network(rng, [3] + [64] * hidden + [4], 6, wl.SELU)
    o_lens, e_lens = lens_pair(cfg)
    o_mesh, e_mesh = meshes_for(cfg, oracle)
    engine = eng.Engine(net, cfg.model, precision=native.SPLIT)
    f = cfg.frames[0]
    got = engine(e_mesh, f["Hoc"], e_lens, f["image"], cfg.fourcc)
    engine.stage([dict(mesh=e_mesh, Hoc=f["Hoc"], lens=e_lens, image=f["image"], fourcc=cfg.fourcc)])
    engine.profile(True)
    engine.run()
    names = [n for n, _, _ in engine.profile_read() if n.startswith("conv")]
    assert len(names) == hidden + 1 and all(n.startswith("conv_bf16_x2_") for n in names[1:hidden]), names
    assert not any("_tobf16_" in n or n.startswith("conv_bf16_bf16_") for n in names), names
    want = o_mesh.classify(f["Hoc"], o_lens, f["image"], cfg.fourcc, vmo.Network(net))
    worst = float(np.abs(got["cls"] - want["cls"]).max())
    print("split, %d hidden layers: worst absolute probability error %.3e" % (hidden, worst), flush=True)
    assert_classification_parity(got, want, PROB_TOL if hidden <= 6 else 2e-4, "split, %d hidden layers" % hidden)


@pytest.mark.parametrize("variant", ["halo8", "fp32_rows_in", "relu_tanh", "selu_last"])
def test_bf16_layer_variants(oracle, variant, monkeypatch):
    """The bf16 layers' less travelled paths on configuration 1's geometry, each within 1e-2 of the fp32 oracle:
    halo8          only 8 halo slots per (half) tile: most neighbours outside a half tile are fetched from global memory;
    fp32_rows_in   the layer before the first bf16 layer writes fp32 rows (the register-gather kernel cannot write hi + lo
                   rows): the bf16 layer splits them at every use;
    relu_tanh      relu and tanh between the layers instead of selu;
    selu_last      a last layer that is not a softmax."""
    if variant == "halo8":
        monkeypatch.setenv("VMHIP_HALO_CAP", "8")
    if variant == "fp32_rows_in":
        monkeypatch.setenv("VMHIP_CONV_KERNEL", "mfma")
    cfg = wl.config(1, n_frames=1)
    rng = np.random.default_rng(77)
    net = wl.glorot_network(rng, [3, 64, 64, 64, 64], 6, wl.SELU)
    if variant == "relu_tanh":
        net = [[(w, b, a if a == wl.SOFTMAX else (wl.RELU if i % 2 == 0 else wl.TANH)) for (w, b, a) in g] for i, g in enumerate(net)]
    if variant == "selu_last":
        net = [[(w, b, wl.SELU) for (w, b, a) in g] for g in net]
    o_lens, e_lens = lens_pair(cfg)
    o_mesh, e_mesh = meshes_for(cfg, oracle)
    engine = eng.Engine(net, cfg.model, precision=native.BF16)
    f = cfg.frames[0]
    got = engine(e_mesh, f["Hoc"], e_lens, f["image"], cfg.fourcc)
    engine.profile(True)
    engine.run()
    names = [n for n, _, _ in engine.profile_read() if n.startswith("conv")]
    first = "conv_mfma_4x64s7" if variant == "fp32_rows_in" else "conv_lds_tox2_4x64s7"
    second = "conv_bf16_f32_tobf16_64x64s7" if variant == "fp32_rows_in" else "conv_bf16_x2_tobf16_64x64s7"
    assert names == [first, second, "conv_bf16_bf16_tox2_64x64s7", "conv_bf16_x2_tof32_64x64s7"], names
    want = o_mesh.classify(f["Hoc"], o_lens, f["image"], cfg.fourcc, vmo.Network(net))
    worst = float(np.abs(got["cls"] - want["cls"]).max())
    print("bf16 %s worst absolute error: %.3e" % (variant, worst), flush=True)
    if variant == "selu_last":  # the outputs are not probabilities: the gate scales with their size
        assert np.array_equal(got["gidx"], want["gidx"]) and np.array_equal(got["nb"], want["nb"])
        assert worst <= BF16_TOL * max(1.0, float(np.abs(want["cls"]).max())), worst
    else:
        assert_classification_parity(got, want, BF16_TOL, "bf16 " + variant)


@pytest.mark.parametrize("variant", ["fp32_rows_in", "relu_tanh", "tanh_only"])
def test_bf16_layer_variants_without_a_rounded_boundary(oracle, variant, monkeypatch):
    """The same less travelled instantiations with every boundary between the bf16 layers as hi + lo pairs
    (VMHIP_BF16_ROUNDED=0): nothing is rounded to bf16 then, so the results must be within 1e-3 of the fp32 oracle - a
    gate that a residual error of a kernel (a wrong operand, a lost register) could not hide behind the way it could
    behind the 1e-2 of a rounded boundary. tanh_only: tanh after every layer, through kernels that read fp32 rows, hi + lo
    rows and write both."""
    monkeypatch.setenv("VMHIP_BF16_ROUNDED", "0")
    if variant == "fp32_rows_in":
        monkeypatch.setenv("VMHIP_CONV_KERNEL", "mfma")
    cfg = wl.config(1, n_frames=1)
    rng = np.random.default_rng(78)
    net = wl.glorot_network(rng, [3, 64, 64, 64, 64, 4], 6, wl.SELU)
    if variant == "relu_tanh":
        net = [[(w, b, a if a == wl.SOFTMAX else (wl.RELU if i % 2 == 0 else wl.TANH)) for (w, b, a) in g] for i, g in enumerate(net)]
    if variant == "tanh_only":
        net = [[(w, b, a if a == wl.SOFTMAX else wl.TANH) for (w, b, a) in g] for g in net]
    o_lens, e_lens = lens_pair(cfg)
    o_mesh, e_mesh = meshes_for(cfg, oracle)
    engine = eng.Engine(net, cfg.model, precision=native.BF16)
    f = cfg.frames[0]
    got = engine(e_mesh, f["Hoc"], e_lens, f["image"], cfg.fourcc)
    engine.profile(True)
    engine.run()
    names = [n for n, _, _ in engine.profile_read() if n.startswith("conv")]
    assert sum(n.startswith("conv_bf16_") for n in names) == 3 and not any("_tobf16_" in n or "_bf16_bf16_" in n for n in names), names
    want = o_mesh.classify(f["Hoc"], o_lens, f["image"], cfg.fourcc, vmo.Network(net))
    worst = float(np.abs(got["cls"] - want["cls"]).max())
    print("bf16 %s without a rounded boundary, worst absolute error: %.3e" % (variant, worst), flush=True)
    assert_classification_parity(got, want, 1e-3, "bf16 " + variant + ", no rounded boundary")


def test_bf16_engine_keeps_narrow_networks_in_fp32(oracle):
    """Rows narrower than 64 channels are not worth bf16 storage (one rounding already costs ~1e-2 on a 3-class
    softmax): a bf16 engine built on configuration 2's network meets the fp32 gate."""
    cfg = wl.config(2, n_frames=1)
    o_lens, e_lens = lens_pair(cfg)
    o_mesh, e_mesh = meshes_for(cfg, oracle)
    engine = eng.Engine(cfg.network, cfg.model, precision=native.BF16)
    f = cfg.frames[0]
    got = engine(e_mesh, f["Hoc"], e_lens, f["image"], cfg.fourcc)
    want = pick(o_mesh, f["Hoc"]).classify(f["Hoc"], o_lens, f["image"], cfg.fourcc, vmo.Network(cfg.network))
    assert_classification_parity(got, want, PROB_TOL, "bf16 engine, narrow network")


@pytest.mark.parametrize("kernel", ["rows", "mfma", "lds", "flow"])
def test_every_convolution_kernel_agrees_with_the_oracle(oracle, kernel, monkeypatch):
    """Every layer shape of configuration 2 through the one-row-per-lane kernel, the matrix-core kernel that
    gathers into registers and the matrix-core kernels that gather from LDS (rows staged through registers /
    loaded straight into LDS / the same without barriers in the tile loop), selected with VMHIP_CONV_KERNEL when the engine is built."""
    monkeypatch.setenv("VMHIP_CONV_KERNEL", kernel)
    cfg = wl.config(2, n_frames=2)
    o_lens, e_lens = lens_pair(cfg)
    o_mesh, e_mesh = meshes_for(cfg, oracle)
    engine = eng.Engine(cfg.network, cfg.model)
    frames = [dict(mesh=e_mesh, Hoc=f["Hoc"], lens=e_lens, image=f["image"], fourcc=cfg.fourcc) for f in cfg.frames]
    engine.profile(False)
    results = engine.classify_batch(frames)
    engine.profile(True)
    engine.run()
    names = [n for n, _, _ in engine.profile_read() if n.startswith("conv")]
    assert len(names) == 8, names
    if kernel == "mfma":
        assert all(n.startswith("conv_mfma_") or n == "conv_rows_16x3s7" for n in names), names
    elif kernel == "flow":  # instantiated for the layers that are bound by the matrix pipe; the rest stay on "lds"
        pre = "conv_%s_" % kernel
        assert [n for n in names if n.startswith(pre)] == [pre + "16x32s7"] + [pre + "32x32s7"] * 4 + [pre + "32x16s7"], names
        assert all(n.startswith((pre, "conv_lds_", "conv_narrow_")) for n in names), names
    else:
        assert all(n.startswith("conv_%s_" % kernel) for n in names), names
    for i, f in enumerate(cfg.frames):
        want = pick(o_mesh, f["Hoc"]).classify(f["Hoc"], o_lens, f["image"], cfg.fourcc, vmo.Network(cfg.network))
        assert_classification_parity(results[i], want, PROB_TOL, "%s frame %d" % (kernel, i))


@pytest.mark.parametrize("kernel", ["lds", "flow"])
@pytest.mark.parametrize("index", [2, 3])
def test_rows_beyond_the_halo_capacity(oracle, index, kernel, monkeypatch):
    """With only 8 halo slots per tile most out-of-tile neighbours are marked as not staged and the LDS kernel
    reads them from global memory: same results (configuration 2's Ring6 and 3's NMGrid8 networks)."""
    monkeypatch.setenv("VMHIP_HALO_CAP", "8")
    monkeypatch.setenv("VMHIP_CONV_KERNEL", kernel)
    cfg = wl.config(index, n_frames=1)
    o_lens, e_lens = lens_pair(cfg)
    o_mesh, e_mesh = meshes_for(cfg, oracle)
    engine = eng.Engine(cfg.network, cfg.model)
    f = cfg.frames[0]
    got = engine(e_mesh, f["Hoc"], e_lens, f["image"], cfg.fourcc)
    engine.profile(True)
    engine.run()
    names = [n for n, _, _ in engine.profile_read() if n.startswith("conv")]
    assert all(n.startswith(("conv_%s_" % kernel, "conv_lds_", "conv_narrow_") if kernel == "flow" else "conv_%s_" % kernel) for n in names), names
    if not (kernel == "flow" and index == 3):  # that kernel has no instantiation for the 24-wide NMGrid8 network
        assert any(n.startswith("conv_%s_" % kernel) for n in names), names
    want = pick(o_mesh, f["Hoc"]).classify(f["Hoc"], o_lens, f["image"], cfg.fourcc, vmo.Network(cfg.network))
    assert_classification_parity(got, want, PROB_TOL, "halo cap 8, cfg%d, %s" % (index, kernel))


@pytest.mark.parametrize("halo_cap", [None, 8], ids=["full halo", "8 halo slots"])
@pytest.mark.parametrize("index", [1, 2, 3])
def test_first_layer_inside_the_neighbourhood_kernel(oracle, index, halo_cap, monkeypatch):
    """The first layer of configurations 1, 2 and 3 (4 -> 16 on Ring6, 4 -> 24 on NMGrid8) is computed by the blocks of the
    neighbourhood kernel for their own tiles; with only 8 halo slots per tile most neighbours outside a tile are read
    from global memory through the table the block has just written. Same results as the oracle, and as the engine
    with the layer as a launch of its own."""
    if halo_cap is not None:
        monkeypatch.setenv("VMHIP_HALO_CAP", str(halo_cap))
    cfg = wl.config(index, n_frames=2 if index == 2 else 1)
    o_lens, e_lens = lens_pair(cfg)
    o_mesh, e_mesh = meshes_for(cfg, oracle)
    engine = eng.Engine(cfg.network, cfg.model)
    frames = [dict(mesh=e_mesh, Hoc=f["Hoc"], lens=e_lens, image=f["image"], fourcc=cfg.fourcc) for f in cfg.frames]
    results = engine.classify_batch(frames)
    monkeypatch.setenv("VMHIP_FUSE_FIRST", "0")  # read when an engine is first used
    apart = eng.Engine(cfg.network, cfg.model)
    engine.profile(True)
    engine.run()
    names = [n for n, _, _ in engine.profile_read()]
    first = "neighbourhood_conv_4x%ds%d" % (cfg.network[0][0][0].shape[1], 7 if index != 3 else 9)
    assert first in names and "neighbourhood" not in names and len([n for n in names if n.startswith("conv")]) == len(cfg.network) - 1, names
    others = apart.classify_batch(frames)
    apart.profile(True)
    apart.run()
    names = [n for n, _, _ in apart.profile_read()]
    assert "neighbourhood" in names and len([n for n in names if n.startswith("conv")]) == len(cfg.network), names
    for i, f in enumerate(cfg.frames):
        want = pick(o_mesh, f["Hoc"]).classify(f["Hoc"], o_lens, f["image"], cfg.fourcc, vmo.Network(cfg.network))
        assert_classification_parity(results[i], want, PROB_TOL, "first layer with the neighbourhood, frame %d" % i)
        assert_classification_parity(others[i], want, PROB_TOL, "first layer apart, frame %d" % i)
        for key in ("px", "gidx", "nb"):
            assert np.array_equal(results[i][key], others[i][key]), key


def test_graph_replays_match_eager_runs(oracle, monkeypatch):
    """A staged batch launches its first run kernel by kernel, captures the second into a HIP graph and replays it
    afterwards. Every replay, with eager work of another engine and synchronisations in between, must reproduce
    the eager results bit for bit (two batches through the same engine, so the graph is rebuilt after restaging)."""
    cfg = wl.config(2, n_frames=3)
    _, e_lens = lens_pair(cfg)
    _, e_mesh = meshes_for(cfg, oracle)
    frames = [dict(mesh=e_mesh, Hoc=f["Hoc"], lens=e_lens, image=f["image"], fourcc=cfg.fourcc) for f in cfg.frames]
    monkeypatch.setenv("VMHIP_GRAPH", "0")
    eager = eng.Engine(cfg.network, cfg.model)
    monkeypatch.setenv("VMHIP_GRAPH", "1")
    graphed = eng.Engine(cfg.network, cfg.model)
    for batch in (frames, frames[:2][::-1]):
        want = eager.classify_batch(batch)
        graphed.stage(batch)
        for replay in range(5):
            graphed.run()
            got = graphed.fetch()
            eager.run()  # unrelated eager work between the replays
            for i in range(len(batch)):
                for key in ("px", "gidx", "nb", "cls"):
                    assert np.array_equal(got[i][key], want[i][key]), "run %d frame %d %s" % (replay, i, key)


def test_a_captured_pass_outlives_the_batch_it_was_captured_with(oracle, monkeypatch):
    """Frame after frame through one engine, the way a camera loop or the pipeline drives it (stage, run once, fetch): the
    first pass is launched kernel by kernel, the second is captured into a HIP graph, and every batch after that - other
    images, other poses, other visible counts, as long as it fits the grids - is a launch of that same graph, its tiles
    in use, frame descriptions and tables read from device memory. Every result is the oracle's. A batch with another
    number of frames, or one that outgrows the grids, is captured again; the pipeline's three engines do the same."""
    monkeypatch.setenv("VMHIP_GRAPH", "1")
    cfg = wl.config(2, n_frames=8)
    o_lens, e_lens = lens_pair(cfg)
    o_mesh, e_mesh = meshes_for(cfg, oracle)
    net = vmo.Network(cfg.network)
    frames = [dict(mesh=e_mesh, Hoc=f["Hoc"], lens=e_lens, image=f["image"], fourcc=cfg.fourcc) for f in cfg.frames]
    wants = [pick(o_mesh, f["Hoc"]).classify(f["Hoc"], o_lens, f["image"], cfg.fourcc, net) for f in cfg.frames]
    # pairs of frames in decreasing order of their candidate counts: the first batch sizes the grids, the others fit
    probe = eng.Engine(cfg.network, cfg.model)
    probe.stage(frames)
    size = [sum(b - a for a, b in probe.staged_ranges(i).reshape(-1, 2)) for i in range(len(frames))]
    order = sorted(range(len(frames)), key=lambda i: -size[i])
    batches = [[order[0], order[1]], [order[2], order[3]], [order[5], order[4]], [order[7], order[6]]]
    engine = eng.Engine(cfg.network, cfg.model)
    for k, b in enumerate(batches):
        engine.stage([frames[i] for i in b])
        engine.run()
        got = engine.fetch()
        for i, r in zip(b, got):
            assert_classification_parity(r, wants[i], PROB_TOL, "batch %d frame %d" % (k, i))
        stats = engine.graph_stats()
        print("after batch %d: %s" % (k, stats), flush=True)
    assert stats == dict(captures=1, graph_launches=3, eager_launches=1), stats
    # the same frames again, the other way round in each batch: still the one graph
    for b in batches:
        engine.stage([frames[i] for i in b[::-1]])
        engine.run()
        for i, r in zip(b[::-1], engine.fetch()):
            assert_classification_parity(r, wants[i], PROB_TOL, "second round frame %d" % i)
    assert engine.graph_stats() == dict(captures=1, graph_launches=7, eager_launches=1), engine.graph_stats()
    # three frames instead of two: another graph (one pass kernel by kernel, then the capture)
    for _ in range(2):
        engine.stage([frames[i] for i in order[:3]])
        engine.run()
        for i, r in zip(order[:3], engine.fetch()):
            assert_classification_parity(r, wants[i], PROB_TOL, "three frames, frame %d" % i)
    stats = engine.graph_stats()
    assert stats["captures"] == 2 and stats["eager_launches"] == 2, stats

    # the pipeline: three engines, each sees every third batch; each launches its first pass kernel by kernel, captures its
    # second and replays from then on
    images = []
    for f in cfg.frames:
        held = native.pinned_empty(f["image"].shape, f["image"].dtype)
        held[...] = f["image"]
        images.append(held)
    pinned = [dict(mesh=e_mesh, Hoc=f["Hoc"], lens=e_lens, image=im, fourcc=cfg.fourcc) for f, im in zip(cfg.frames, images)]
    pipe = eng.Pipeline(cfg.network, cfg.model)
    sequence = [[order[0], order[1]]] * 3 + [[order[2], order[3]], [order[4], order[5]], [order[6], order[7]]] * 3
    got = []
    for b in sequence:
        done = pipe.submit([pinned[i] for i in b])
        if done is not None:
            got.append([{k: v.copy() for k, v in r.items()} for r in done])
    while True:
        done = pipe.flush()
        if done is None:
            break
        got.append([{k: v.copy() for k, v in r.items()} for r in done])
    assert len(got) == len(sequence)
    for b, results in zip(sequence, got):
        for i, r in zip(b, results):
            assert_classification_parity(r, wants[i], PROB_TOL, "pipeline frame %d" % i)
    stats = pipe.graph_stats()
    assert stats == dict(captures=3, graph_launches=len(sequence) - 3, eager_launches=3), stats


def test_graph_replays_with_event_records_match_eager_runs(oracle, monkeypatch):
    """Timing mode 2 (events around the launches of the longest kernel only) keeps the pass in its captured graph: the
    event records are nodes of it. Every replay must reproduce the eager results bit for bit, and every replay's
    events must give a duration of that kernel that fits inside the pass's wall time."""
    import time
    cfg = wl.config(2, n_frames=3)
    _, e_lens = lens_pair(cfg)
    _, e_mesh = meshes_for(cfg, oracle)
    frames = [dict(mesh=e_mesh, Hoc=f["Hoc"], lens=e_lens, image=f["image"], fourcc=cfg.fourcc) for f in cfg.frames]
    monkeypatch.setenv("VMHIP_GRAPH", "0")
    eager = eng.Engine(cfg.network, cfg.model)
    want = eager.classify_batch(frames)
    monkeypatch.setenv("VMHIP_GRAPH", "1")
    timed = eng.Engine(cfg.network, cfg.model)
    timed.stage(frames)
    timed.profile(1)
    timed.run()
    every_kernel = timed.profile_read()
    longest = max(set(name for name, ms, units in every_kernel), key=lambda k: sum(ms for name, ms, units in every_kernel if name == k))
    timed.profile(2)
    for replay in range(6):  # one run kernel by kernel, one that is captured, then replays
        t0 = time.perf_counter()
        timed.run()
        wall_ms = (time.perf_counter() - t0) * 1e3
        slots = timed.profile_read()
        assert slots and all(name == longest for name, ms, units in slots)
        assert all(ms > 0 for name, ms, units in slots) and sum(ms for name, ms, units in slots) < wall_ms
        got = timed.fetch()
        eager.run()  # unrelated eager work between the replays
        for i in range(len(frames)):
            for key in ("px", "gidx", "nb", "cls"):
                assert np.array_equal(got[i][key], want[i][key]), "run %d frame %d %s" % (replay, i, key)
    timed.profile(0)
    timed.run()  # and back to the graph without events
    got = timed.fetch()
    for i in range(len(frames)):
        assert np.array_equal(got[i]["cls"], want[i]["cls"])


def _example_network():
    import json
    import os
    here = os.path.dirname(os.path.abspath(__file__))
    fixture = np.load(os.path.join(here, "golden", "example_model.npz"))
    meta = json.load(open(os.path.join(here, "golden", "example_poses.json")))
    network = []
    for g, l, act in fixture["activations"]:
        while len(network) <= g:
            network.append([])
        network[g].append((fixture["w_%d_%d" % (g, l)], fixture["b_%d_%d" % (g, l)], int(act)))
    return network, meta


def test_reference_example_network_on_its_dataset_poses(oracle):
    """The reference's exported example network (example/model.yaml: 4->16, 16->16 x5, 16->8, 8->8 x5, 8->5) on the
    lens and camera pose of its dataset elements (example/images/lens*.yaml, rectilinear 1280x1024), with synthetic
    BGRA images: projection and probabilities on all 30 poses, classified in one batch."""
    network, meta = _example_network()
    assert meta["mesh"] == "RING6" and meta["shape"] == "SPHERE"
    heights = [p["Hoc"][2][3] for p in meta["poses"]]  # 0.78 m to 1.2 m: one mesh per height band, as the reference does
    mesh_args = (wl.RING6, wl.SPHERE, meta["radius"], min(heights), max(heights), 6.0, 0.5, 15.0)
    o_mesh = oracle.visualmesh(*mesh_args)
    e_mesh = eng.VisualMesh(*mesh_args)
    engine = eng.Engine(network, wl.RING6)
    rng = np.random.default_rng(77)
    projections = {"RECTILINEAR": wl.RECTILINEAR, "EQUISOLID": wl.EQUISOLID, "EQUIDISTANT": wl.EQUIDISTANT}
    views = []
    for p in meta["poses"]:
        args = (p["width"], p["height"], projections[p["projection"]], p["focal_length"], p["fov"], tuple(p["centre"]), tuple(p["k"]))
        views.append((np.array(p["Hoc"], np.float32), vmo.make_lens(*args), native.make_lens(*args), p))
    for Hoc, o_lens, e_lens, p in views:
        assert_projection_parity(engine(e_mesh, Hoc, e_lens), pick(o_mesh, Hoc).project(Hoc, o_lens), "example pose " + p["number"])
    chosen = views
    images = [wl.random_image(rng, p["width"], p["height"], 4) for _, _, _, p in chosen]
    frames = [dict(mesh=e_mesh, Hoc=H, lens=el, image=im, fourcc=wl.fourcc("BGRA")) for (H, _, el, _), im in zip(chosen, images)]
    results = engine.classify_batch(frames)
    engine.profile(True)
    engine.run()
    names = [n for n, _, _ in engine.profile_read() if "conv" in n]
    # the first layer rides on the neighbourhood kernel, the other twelve gather from LDS
    assert len(names) == 13 and names[0] == "neighbourhood_conv_4x16s7" and all(n.startswith("conv_lds_") for n in names[1:]), names
    for (H, ol, _, p), im, got in zip(chosen, images, results):
        want = pick(o_mesh, H).classify(H, ol, im, wl.fourcc("BGRA"), vmo.Network(network))
        print("example pose", p["number"], "V =", len(want["gidx"]), flush=True)
        assert got["cls"].shape[1] == 5
        assert_classification_parity(got, want, PROB_TOL, "example pose " + p["number"])


def test_mesh_cache_is_bounded_and_keeps_staged_meshes(oracle):
    """The device mesh cache releases least recently used meshes beyond its byte limit, never one the staged batch
    uses, and a mesh that comes back is uploaded again with unchanged results."""
    cfg = wl.config(1, n_frames=1)
    o_lens, e_lens = lens_pair(cfg)
    f = cfg.frames[0]
    heights = (1.2, 1.0, 0.9)
    args = [(cfg.model, cfg.shape, cfg.radius, h, cfg.k, cfg.max_distance) for h in heights]
    meshes = [eng.Mesh(*a) for a in args]
    engine = eng.Engine(cfg.network, cfg.model)
    Hocs = []
    for h in heights:
        H = np.array(f["Hoc"], np.float32).copy()
        H[2][3] = h
        Hocs.append(H)
    one = meshes[0].n_nodes * (12 + 4 * meshes[0].n_neighbours)
    engine.set_cache_limit(int(2.5 * one))  # room for two of the three (they are of similar size)
    want = [oracle.mesh(*a).project(H, o_lens) for a, H in zip(args, Hocs)]
    for m, H, w in zip(meshes, Hocs, want):
        assert_projection_parity(engine(m, H, e_lens), w, "first visit")
    n, nbytes = engine.cache_info()
    assert n == 2 and nbytes <= 2.5 * one, (n, nbytes)
    assert_projection_parity(engine(meshes[0], Hocs[0], e_lens), want[0], "mesh that had been released")
    # a staged batch pins its mesh whatever the limit
    engine.stage([dict(mesh=meshes[1], Hoc=Hocs[1], lens=e_lens, image=f["image"], fourcc=cfg.fourcc)])
    engine.set_cache_limit(1)
    engine(meshes[0], Hocs[0], e_lens)
    engine(meshes[2], Hocs[2], e_lens)
    engine.run()
    got = engine.fetch()[0]
    assert_projection_parity(got, want[1], "staged mesh after other meshes went through a full cache")
    n, _ = engine.cache_info()
    assert n == 2, n  # the staged mesh and the last one used


@pytest.mark.parametrize("arg_max_only", [False, True])
def test_detections_and_clusters_on_the_device(oracle, arg_max_only):
    """vmhip_batch_detect against the same selection and clustering done on the host from the full download of the same
    run: the detected nodes (order, mesh indices, pixels, probabilities) must be identical, and the clusters must be
    the connected components scipy finds in the neighbourhood graph restricted to the detections, numbered by their
    first detection; sizes and bounding boxes exact, centres to rounding. (The probabilities themselves are checked
    against the oracle by the tests above; here both sides start from the same device results.)"""
    import scipy.sparse as sp
    from scipy.sparse.csgraph import connected_components
    cfg = wl.config(2, n_frames=3)
    _, e_lens = lens_pair(cfg)
    _, e_mesh = meshes_for(cfg, oracle)
    engine = eng.Engine(cfg.network, cfg.model)
    frames = [dict(mesh=e_mesh, Hoc=f["Hoc"], lens=e_lens, image=f["image"], fourcc=cfg.fourcc) for f in cfg.frames]
    engine.stage(frames)
    engine.run()
    full = engine.fetch()
    n_classes = full[0]["cls"].shape[1]
    assert n_classes == 3
    seen = dict(detections=0, clusters=0, largest=0)
    for cls, thr in [(1, 0.34), (0, 0.5), (2, 0.9999)]:
        got = engine.detect(cls, thr, arg_max_only=arg_max_only, clusters=True)
        assert len(got) == len(full)
        for f, (g, r) in enumerate(zip(got, full)):
            V = len(r["gidx"])
            p = r["cls"][:V]
            hit = p[:, cls] >= np.float32(thr)
            if arg_max_only:
                hit &= np.argmax(p, axis=1) == cls  # numpy's argmax takes the first maximum too
            rows = np.nonzero(hit)[0]
            what = "class %d threshold %g frame %d" % (cls, thr, f)
            assert len(g["node"]) == len(rows), what
            np.testing.assert_array_equal(g["node"], r["gidx"][rows], what)
            np.testing.assert_array_equal(g["pixel"], r["px"][rows], what)
            np.testing.assert_array_equal(g["probability"], p[rows, cls], what)
            # connected components of the detections under the (directed) neighbourhood table, taken as undirected
            det_of_row = -np.ones(V + 1, np.int64)
            det_of_row[rows] = np.arange(len(rows))
            nb = r["nb"][rows]                      # [n_det, nn] local rows, V = not visible
            src = np.repeat(np.arange(len(rows)), nb.shape[1])
            dst = det_of_row[nb.reshape(-1)]
            keep = dst >= 0
            graph = sp.coo_matrix((np.ones(keep.sum()), (src[keep], dst[keep])), shape=(len(rows), len(rows)))
            n_comp, label = connected_components(graph, directed=False)
            assert len(g["cluster_size"]) == n_comp, what
            if len(rows) == 0:
                continue
            # renumber scipy's labels by first appearance
            first = np.full(n_comp, len(rows))
            np.minimum.at(first, label, np.arange(len(rows)))
            order = np.argsort(first)
            renumber = np.empty(n_comp, np.int64)
            renumber[order] = np.arange(n_comp)
            want_cluster = renumber[label]
            seen["detections"] += len(rows)
            seen["clusters"] += n_comp
            seen["largest"] = max(seen["largest"], int(np.bincount(want_cluster).max()))
            np.testing.assert_array_equal(g["cluster"], want_cluster, what)
            np.testing.assert_array_equal(g["cluster_size"], np.bincount(want_cluster, minlength=n_comp), what)
            px = r["px"][rows]
            for c in range(n_comp):
                m = px[want_cluster == c]
                np.testing.assert_array_equal(g["cluster_box"][c], [m[:, 0].min(), m[:, 1].min(), m[:, 0].max(), m[:, 1].max()], what)
                np.testing.assert_allclose(g["cluster_centre"][c], m.astype(np.float64).mean(axis=0), rtol=1e-5, err_msg=what)
    # the cases are not trivial: many detections, many clusters, clusters of more than a handful of nodes
    assert seen["detections"] > 1000 and seen["clusters"] > 100 and seen["largest"] > 8, seen
    # without clustering only the detections come back
    got = engine.detect(1, 0.34, arg_max_only=arg_max_only, clusters=False)
    assert all(len(g["cluster_size"]) == 0 and len(g["cluster"]) == 0 for g in got)
    # a class the network does not have
    with pytest.raises(RuntimeError):
        engine.detect(3, 0.5)


def test_a_wait_that_runs_out_fails_the_run(oracle):
    """The barrier-free convolution kernel bounds every wait by a poll count. With the count set to one poll (from the
    host; the kernels still end normally: a wave whose wait runs out tells its block and leaves its tile loop, and so
    does every wave that sees the flag) the run must be reported as failed, and with the count restored the same staged
    batch must run and give the oracle's results."""
    cfg = wl.config(2, n_frames=1)
    o_lens, e_lens = lens_pair(cfg)
    o_mesh, e_mesh = meshes_for(cfg, oracle)
    engine = eng.Engine(cfg.network, cfg.model)
    f = cfg.frames[0]
    frames = [dict(mesh=e_mesh, Hoc=f["Hoc"], lens=e_lens, image=f["image"], fourcc=cfg.fourcc)]
    engine.stage(frames)
    lib = native.hip()
    native.hip_check(lib.vmhip_debug_set(native.DEBUG_FLOW_POLL_LIMIT, 1))
    try:
        with pytest.raises(RuntimeError, match="gave up waiting"):
            engine.run()
        # a failed run leaves nothing to fetch
        with pytest.raises(RuntimeError):
            engine.fetch()
    finally:
        native.hip_check(lib.vmhip_debug_set(native.DEBUG_FLOW_POLL_LIMIT, 0))
    engine.run()  # the failed run reset the batch's count of such waits, or this one would fail too
    got = engine.fetch()[0]
    want = pick(o_mesh, f["Hoc"]).classify(f["Hoc"], o_lens, f["image"], cfg.fourcc, vmo.Network(cfg.network))
    assert_classification_parity(got, want, PROB_TOL, "after a failed run")


def test_images_in_page_locked_memory(oracle):
    """vmhip_host_alloc: an image that lies in page-locked memory is staged from there and gives the same results."""
    cfg = wl.config(1)
    o_lens, e_lens = lens_pair(cfg)
    o_mesh, e_mesh = meshes_for(cfg, oracle)
    engine = eng.Engine(cfg.network, cfg.model)
    f = cfg.frames[0]
    image = native.pinned_empty(f["image"].shape, f["image"].dtype)
    image[...] = f["image"]
    got = engine(e_mesh, f["Hoc"], e_lens, image, cfg.fourcc)
    want = pick(o_mesh, f["Hoc"]).classify(f["Hoc"], o_lens, f["image"], cfg.fourcc, vmo.Network(cfg.network))
    assert_classification_parity(got, want, PROB_TOL, "image in page-locked memory")
    del image  # frees the allocation (the owner goes with the last view)


def test_run_in_two_halves_and_two_engines_overlapping(oracle):
    """vmhip_batch_run_async / vmhip_batch_wait: two engines take turns, each staging its frames while the other's pass is
    in flight; results must equal the oracle's, and a batch in flight must refuse to be staged, run or read."""
    cfg = wl.config(2, n_frames=4)
    o_lens, e_lens = lens_pair(cfg)
    o_mesh, e_mesh = meshes_for(cfg, oracle)
    engines = [eng.Engine(cfg.network, cfg.model), eng.Engine(cfg.network, cfg.model)]
    halves = [cfg.frames[:2], cfg.frames[2:]]
    staged = [[dict(mesh=e_mesh, Hoc=f["Hoc"], lens=e_lens, image=f["image"], fourcc=cfg.fourcc) for f in h] for h in halves]
    engines[0].stage(staged[0])
    engines[0].run_async()
    with pytest.raises(RuntimeError, match="in flight"):
        engines[0].run_async()
    with pytest.raises(RuntimeError, match="in flight"):
        engines[0].stage(staged[0])
    with pytest.raises(RuntimeError):
        engines[0].fetch()            # no completed run yet
    engines[1].stage(staged[1])       # overlaps the pass of engine 0
    engines[1].run_async()
    engines[0].wait()
    got0 = engines[0].fetch()
    engines[0].stage(staged[0])       # and again the other way round
    engines[0].run_async()
    engines[1].wait()
    got1 = engines[1].fetch()
    engines[0].wait()
    again0 = engines[0].fetch()
    with pytest.raises(RuntimeError, match="no run in flight"):
        engines[0].wait()
    net = vmo.Network(cfg.network)
    for got, frames in ((got0, halves[0]), (got1, halves[1]), (again0, halves[0])):
        for g, f in zip(got, frames):
            want = pick(o_mesh, f["Hoc"]).classify(f["Hoc"], o_lens, f["image"], cfg.fourcc, net)
            assert_classification_parity(g, want, PROB_TOL, "two engines taking turns")


@pytest.mark.parametrize("index,n_frames", [(2, 6), (3, 2), (1, 2)])
def test_lookup_on_the_device_gives_the_hosts_ranges(oracle, index, n_frames):
    """The walk of the cone tree on the device (vmhip_frame.lookup) must cover exactly the nodes the host's walk covers:
    the staged ranges are compared pair by pair with Mesh::lookup's, and the classification that follows with the
    oracle's. Configuration 2 has frames at many pitches and several meshes, 3 a rectilinear lens (edge planes
    instead of edge cones)."""
    cfg = wl.config(index, n_frames=n_frames)
    o_lens, e_lens = lens_pair(cfg)
    o_mesh, e_mesh = meshes_for(cfg, oracle)
    engine = eng.Engine(cfg.network, cfg.model)
    engine.set_device_lookup(True)
    frames = [dict(mesh=e_mesh, Hoc=f["Hoc"], lens=e_lens, image=f["image"], fourcc=cfg.fourcc) for f in cfg.frames]
    engine.stage(frames)
    for i, f in enumerate(cfg.frames):
        want = engine._pick(e_mesh, f["Hoc"]).lookup(f["Hoc"], e_lens)
        got = engine.staged_ranges(i)
        print(cfg.name, "frame", i, "ranges", len(want), flush=True)
        assert np.array_equal(got, want), "ranges of frame %d differ" % i
    engine.run()
    results = engine.fetch()
    net = vmo.Network(cfg.network)
    for i, f in enumerate(cfg.frames):
        want = pick(o_mesh, f["Hoc"]).classify(f["Hoc"], o_lens, f["image"], cfg.fourcc, net)
        assert_classification_parity(results[i], want, PROB_TOL, "%s frame %d, lookup on the device" % (cfg.name, i))
    # and back: the same engine with the host's lookup stages the same ranges
    engine.set_device_lookup(False)
    engine.stage(frames)
    for i, f in enumerate(cfg.frames):
        assert np.array_equal(engine.staged_ranges(i), engine._pick(e_mesh, f["Hoc"]).lookup(f["Hoc"], e_lens))


@pytest.mark.parametrize("index,n_frames", [(2, 3), (3, 1)])
def test_lookup_graph_export(oracle, index, n_frames):
    """vmhip_batch_export against the oracle's restatement of the LookupVisualMesh op: vectors and graph bit-exact for
    HARD and SAME edges; the pixel of every exported node within 1e-3 px of the oracle's projection of its vector
    (all visible ones through the projected mesh, a sample of the others one by one)."""
    cfg = wl.config(index, n_frames=n_frames)
    o_lens, e_lens = lens_pair(cfg)
    o_mesh, e_mesh = meshes_for(cfg, oracle)
    engine = eng.Engine(cfg.network, cfg.model)
    engine.stage([dict(mesh=e_mesh, Hoc=f["Hoc"], lens=e_lens, image=f["image"], fourcc=cfg.fourcc) for f in cfg.frames])
    for i, f in enumerate(cfg.frames):
        mesh = pick(o_mesh, f["Hoc"])
        want = mesh.lookup_graph(f["Hoc"], o_lens)
        got = engine.lookup_graph(i)
        print(cfg.name, "frame", i, "points", len(want["gidx"]), flush=True)
        assert np.array_equal(got["vectors"], want["vectors"])
        assert np.array_equal(got["graph"], want["graph"])
        assert (want["graph"] < 0).any(), "the frame must cut the mesh for the edges to matter"
        assert np.array_equal(engine.lookup_graph(i, same_edges=True)["graph"], mesh.lookup_graph(f["Hoc"], o_lens, same_edges=True)["graph"])
        projected = mesh.project(f["Hoc"], o_lens)
        rows = np.searchsorted(want["gidx"], projected["gidx"])
        assert np.abs(got["px"][rows] - projected["px"]).max() <= 1e-3
        Rco = np.asarray(f["Hoc"], np.float32)[:3, :3].T
        for r in np.linspace(0, len(want["gidx"]) - 1, 200).astype(int):
            v = want["vectors"][r]
            cam = np.array([Rco[k, 2] * v[2] + (Rco[k, 1] * v[1] + Rco[k, 0] * v[0]) for k in range(3)], np.float32)
            assert np.abs(oracle.fn_project(cam, o_lens) - got["px"][r]).max() <= 1e-3


def test_results_into_page_locked_memory(oracle):
    """vmhip_batch_fetch into arrays from vmhip_host_alloc gives the results of the ordinary fetch, also when the arrays
    are reused by a second, smaller batch."""
    cfg = wl.config(2, n_frames=3)
    o_lens, e_lens = lens_pair(cfg)
    o_mesh, e_mesh = meshes_for(cfg, oracle)
    engine = eng.Engine(cfg.network, cfg.model)
    frames = [dict(mesh=e_mesh, Hoc=f["Hoc"], lens=e_lens, image=f["image"], fourcc=cfg.fourcc) for f in cfg.frames]
    for chosen in (frames, frames[1:2]):
        engine.stage(chosen)
        engine.run()
        plain = engine.fetch()
        pinned = engine.fetch_pinned()
        assert len(plain) == len(pinned) == len(chosen)
        for a, b in zip(plain, pinned):
            assert len(a["gidx"]) > 1000
            for key in ("px", "nb", "gidx", "cls"):
                assert np.array_equal(a[key], b[key]), key
        # the same as one transfer: gathered into one block on the device, one copy, views into the block
        packed = engine.fetch_packed()
        assert len(packed) == len(chosen)
        for a, b in zip(plain, packed):
            for key in ("px", "nb", "gidx", "cls"):
                assert a[key].dtype == b[key].dtype and np.array_equal(a[key], b[key]), key


def test_pipeline_of_three_engines(oracle):
    """Pipeline<float>: batches of different sizes through submit() (one frame that sees nothing among them), the results
    of batch k come back from the submit of batch k + 2 or from flush(), every one the oracle's; a single batch drains
    with flush() alone."""
    cfg = wl.config(2, n_frames=7)
    o_lens, e_lens = lens_pair(cfg)
    o_mesh, e_mesh = meshes_for(cfg, oracle)
    net = vmo.Network(cfg.network)
    images = []
    for f in cfg.frames:
        held = native.pinned_empty(f["image"].shape, f["image"].dtype)
        held[...] = f["image"]
        images.append(held)
    frames = [dict(mesh=e_mesh, Hoc=f["Hoc"], lens=e_lens, image=im, fourcc=cfg.fourcc) for f, im in zip(cfg.frames, images)]
    up = dict(mesh=e_mesh, Hoc=wl.make_hoc(1.0, math.radians(-85), 0.0, 0.0), lens=native.make_lens(1280, 1024, wl.RECTILINEAR, 700.0, 1.6),
              image=images[0], fourcc=cfg.fourcc)
    wants = [pick(o_mesh, f["Hoc"]).classify(f["Hoc"], o_lens, f["image"], cfg.fourcc, net) for f in cfg.frames]
    batches = [[0, 1], [2], [3, "up", 4], [5, 6], [1]]
    pipe = eng.Pipeline(cfg.network, cfg.model)
    got = []
    for b in batches:
        done = pipe.submit([up if i == "up" else frames[i] for i in b])
        if done is not None:
            got.append([{k: v.copy() for k, v in r.items()} for r in done])
    assert len(got) == len(batches) - 2
    while True:
        done = pipe.flush()
        if done is None:
            break
        got.append([{k: v.copy() for k, v in r.items()} for r in done])
    assert len(got) == len(batches)
    for b, results in zip(batches, got):
        assert len(results) == len(b)
        for i, r in zip(b, results):
            if i == "up":
                assert len(r["gidx"]) == 0
            else:
                assert_classification_parity(r, wants[i], PROB_TOL, "pipeline frame %d" % i)
    single = eng.Pipeline(cfg.network, cfg.model)
    assert single.submit([frames[0]]) is None
    done = single.flush()
    assert done is not None and single.flush() is None
    assert_classification_parity(done[0], wants[0], PROB_TOL, "pipeline of one batch")


def test_packed_fetch_of_mixed_frames(oracle):
    """vmhip_batch_fetch_packed_async on a batch whose frames differ in lens and view, with a frame that sees nothing in
    the middle, and after a projection-only run (no classifications)."""
    rng = np.random.default_rng(4)
    lens = native.make_lens(320, 256, wl.EQUISOLID, 105.0, math.pi)
    m6 = eng.Mesh(wl.RING6, wl.SPHERE, 0.0949, 1.0, 3.0, 8.0)
    img = wl.random_image(rng, 320, 256, 4)
    down = wl.make_hoc(1.0, math.radians(35), 0.03, -0.02)
    narrow = native.make_lens(320, 256, wl.RECTILINEAR, 175.0, 1.9)
    up = wl.make_hoc(1.0, math.radians(-80), 0.0, 0.0)
    engine = eng.Engine([], wl.RING6)
    frames = [dict(mesh=m6, Hoc=down, lens=lens, image=img, fourcc=wl.fourcc("RGBA")),
              dict(mesh=m6, Hoc=up, lens=narrow, image=img, fourcc=wl.fourcc("RGBA")),
              dict(mesh=m6, Hoc=wl.make_hoc(1.0, math.radians(50), 0.0, 0.3), lens=lens, image=img, fourcc=wl.fourcc("RGBA"))]
    engine.stage(frames)
    engine.run()
    plain, packed = engine.fetch(), engine.fetch_packed()
    assert len(plain[1]["gidx"]) == 0 and len(packed[1]["gidx"]) == 0 and len(plain[0]["gidx"]) > 100
    for a, b in zip(plain, packed):
        for key in ("px", "nb", "gidx", "cls"):
            assert np.array_equal(a[key], b[key]), key


@pytest.mark.parametrize("stage_waits", [True, False], ids=["stage", "stage_async"])
def test_fetch_in_two_halves_and_three_engines_in_rotation(oracle, stage_waits):
    """vmhip_batch_fetch_async / vmhip_batch_fetch_wait: three engines in rotation, one staging, one running and one
    copying its results out at any time; every batch must give the oracle's results, and a batch whose fetch is in
    flight must refuse to be staged, run or fetched again. With stage_async the uploads are only queued (from page-locked
    images) and a batch staged twice in a row must end up with the second set of frames."""
    cfg = wl.config(2, n_frames=6)
    o_lens, e_lens = lens_pair(cfg)
    o_mesh, e_mesh = meshes_for(cfg, oracle)
    engines = [eng.Engine(cfg.network, cfg.model) for _ in range(3)]
    groups = [cfg.frames[0:2], cfg.frames[2:4], cfg.frames[4:6]]
    images = {}
    for g in groups:
        for f in g:
            held = native.pinned_empty(f["image"].shape, f["image"].dtype)
            held[...] = f["image"]
            images[id(f)] = held
    staged = [[dict(mesh=e_mesh, Hoc=f["Hoc"], lens=e_lens, image=images[id(f)], fourcc=cfg.fourcc) for f in g] for g in groups]
    net = vmo.Network(cfg.network)
    wants = [[pick(o_mesh, f["Hoc"]).classify(f["Hoc"], o_lens, f["image"], cfg.fourcc, net) for f in g] for g in groups]
    results = {}
    pending = {}
    for step in range(3 + 2):          # every engine's group once, then the pipeline drains
        if step < 3:
            e = engines[step]
            if not stage_waits and step == 0:
                e.stage(staged[2], wait=False)  # overwritten by the next stage before any run
            e.stage(staged[step], wait=stage_waits)
            e.run_async()
        if 1 <= step <= 3:
            e = engines[step - 1]
            e.wait()
            pending[step - 1] = e.fetch_pinned(wait=False)
            if step == 1:
                with pytest.raises(RuntimeError, match="fetch of this batch is still in flight"):
                    e.run()
                with pytest.raises(RuntimeError, match="fetch of this batch is still in flight"):
                    e.stage(staged[0])
                with pytest.raises(RuntimeError, match="fetch of this batch is still in flight"):
                    e.fetch()
        if step >= 2:
            e = engines[step - 2]
            e.fetch_wait()
            results[step - 2] = pending.pop(step - 2)
    with pytest.raises(RuntimeError, match="no fetch in flight"):
        engines[0].fetch_wait()
    for g in range(3):
        for got, want in zip(results[g], wants[g]):
            assert_classification_parity(got, want, PROB_TOL, "group %d of the rotation" % g)

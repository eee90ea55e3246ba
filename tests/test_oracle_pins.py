"""Pins of the CPU oracle that need nothing from the reference: closed forms, invariants, special cases that
reduce to textbook formulas, and brute force on small inputs. Each is chosen so that a plausible mistake (a
dropped term, a wrong sign or index, swapped operands or kernels) fails it."""
import math

import numpy as np
import pytest

from oracle import vmo
from visualmesh_amd import workloads as wl

LENSES = {
    "rectilinear": (1280, 1024, wl.RECTILINEAR, 700.0, math.pi / 2),
    "equisolid": (1280, 1024, wl.EQUISOLID, 420.0, math.pi),
    "equidistant": (2048, 1536, wl.EQUIDISTANT, 672.0, math.pi),
}


# ------------------------------------------------------------------ projection
@pytest.mark.parametrize("name", sorted(LENSES))
def test_optical_axis_projects_to_image_centre_minus_lens_centre(oracle, name):
    W, H, proj, f, fov = LENSES[name]
    lens = vmo.make_lens(W, H, proj, f, fov, centre=(7.5, -3.25))
    px = oracle.fn_project((1.0, 0.0, 0.0), lens)
    assert px[0] == W * 0.5 - 7.5 and px[1] == H * 0.5 + 3.25


@pytest.mark.parametrize("name", sorted(LENSES))
def test_radius_follows_the_textbook_lens_formula(oracle, name):
    """camera x forward, y left, z up; image x right, y down: a ray to the left lands left of centre, a ray
    upwards lands above it, at radius f*tan(t), 2f*sin(t/2) or f*t."""
    W, H, proj, f, fov = LENSES[name]
    lens = vmo.make_lens(W, H, proj, f, fov)
    rng = np.random.default_rng(0)
    for _ in range(200):
        t = rng.uniform(0.01, 0.7)
        a = rng.uniform(0, 2 * math.pi)
        ray = (math.cos(t), math.sin(t) * math.cos(a), math.sin(t) * math.sin(a))
        r = {wl.RECTILINEAR: f * math.tan(t), wl.EQUISOLID: 2 * f * math.sin(t / 2), wl.EQUIDISTANT: f * t}[proj]
        want = (W / 2 - r * math.cos(a), H / 2 - r * math.sin(a))
        px = oracle.fn_project(np.array(ray, np.float32), lens)
        assert abs(px[0] - want[0]) < 2e-3 and abs(px[1] - want[1]) < 2e-3


def test_rectilinear_is_a_pinhole(oracle):
    lens = vmo.make_lens(1280, 1024, wl.RECTILINEAR, 700.0, math.pi / 2)
    for ray in [(0.9, 0.3, -0.2), (0.8, -0.1, 0.5), (0.99, 0.05, 0.02)]:
        v = np.array(ray) / np.linalg.norm(ray)
        px = oracle.fn_project(v.astype(np.float32), lens)
        assert abs(px[0] - (640 - 700 * v[1] / v[0])) < 2e-3 and abs(px[1] - (512 - 700 * v[2] / v[0])) < 2e-3


@pytest.mark.parametrize("name", sorted(LENSES))
def test_project_inverts_unproject(oracle, name):
    W, H, proj, f, fov = LENSES[name]
    lens = vmo.make_lens(W, H, proj, f, fov, centre=(4.0, -6.0))
    rng = np.random.default_rng(1)
    for _ in range(200):
        px = (rng.uniform(0, W), rng.uniform(0, H))
        ray = oracle.fn_unproject(px, lens)
        assert abs(np.linalg.norm(ray) - 1) < 1e-5
        back = oracle.fn_project(ray, lens)
        assert abs(back[0] - px[0]) < 5e-3 and abs(back[1] - px[1]) < 5e-3


def test_distortion_polynomial_against_float64(oracle):
    """r_d = r(1 - k1 r^2 + (3 k1^2 - k2) r^4 + (-12 k1^3 + 8 k1 k2) r^6 + (55 k1^4 - 55 k1^2 k2 + 5 k2^2) r^8),
    the published inverse radial distortion series truncated after four terms."""
    k1, k2 = -1.2e-7, 3.0e-14
    lens = vmo.make_lens(1280, 1024, wl.EQUIDISTANT, 400.0, math.pi, k=(k1, k2))
    for t in (0.1, 0.5, 1.0, 1.4):
        ray = np.array((math.cos(t), math.sin(t), 0.0), np.float32)
        r = 400.0 * math.acos(float(ray[0]))
        rd = r * (1 - k1 * r**2 + (3 * k1**2 - k2) * r**4 + (-12 * k1**3 + 8 * k1 * k2) * r**6
                  + (55 * k1**4 - 55 * k1**2 * k2 + 5 * k2**2) * r**8)
        px = oracle.fn_project(ray, lens)
        assert abs(px[0] - (640 - rd)) < 2e-3 and abs(px[1] - 512) < 1e-3


# ------------------------------------------------------------------ sampling
def test_bilinear_at_integer_coordinates_is_the_texel(oracle):
    rng = np.random.default_rng(2)
    W, H = 32, 24
    img = wl.random_image(rng, W, H, 4)
    px4 = img.reshape(H, W, 4)
    for (x, y) in [(0, 0), (5, 7), (30, 22), (17, 3)]:
        got = oracle.fn_interpolate((float(x), float(y)), img, W, H, wl.fourcc("RGBA"))
        assert np.array_equal(got, px4[y, x].astype(np.float32) * np.float32(1.0 / 255.0))
        got = oracle.fn_interpolate((float(x), float(y)), img, W, H, wl.fourcc("BGRA"))
        assert np.array_equal(got, px4[y, x, [2, 1, 0, 3]].astype(np.float32) * np.float32(1.0 / 255.0))


def test_bilinear_against_float64_and_channel_orders(oracle):
    rng = np.random.default_rng(3)
    W, H = 40, 30
    for code, bpp, order in (("RGBA", 4, [0, 1, 2, 3]), ("BGRA", 4, [2, 1, 0, 3]), ("RGB3", 3, [0, 1, 2]), ("BGR3", 3, [2, 1, 0]),
                             ("GRAY", 1, [0, 0, 0])):
        img = wl.random_image(rng, W, H, bpp)
        t = img.reshape(H, W, bpp).astype(np.float64) / 255.0
        for _ in range(100):
            x, y = rng.uniform(0, W - 1.001), rng.uniform(0, H - 1.001)
            x0, y0 = int(math.floor(x)), int(math.floor(y))
            fx, fy = x - x0, y - y0
            want = ((t[y0, x0] * (1 - fx) + t[y0, x0 + 1] * fx) * (1 - fy) + (t[y0 + 1, x0] * (1 - fx) + t[y0 + 1, x0 + 1] * fx) * fy)[order]
            got = oracle.fn_interpolate((x, y), img, W, H, wl.fourcc(code))
            assert np.abs(got[:len(order)] - want).max() < 1e-5
            if bpp != 4:
                assert abs(got[3] - 1.0) < 1e-6  # formats without alpha report 1


def test_unsupported_fourcc_is_rejected(oracle):
    with pytest.raises(ValueError):
        oracle.fn_interpolate((1.0, 1.0), np.zeros((4, 4), np.uint8), 4, 4, wl.fourcc("NV12"))


MHC = {  # Malvar-He-Cutler 5x5 filters x64, as published (IPOL 2011, "Malvar-He-Cutler Linear Image Demosaicking")
    "G_at_RB": [[0, 0, -8, 0, 0], [0, 0, 16, 0, 0], [-8, 16, 32, 16, -8], [0, 0, 16, 0, 0], [0, 0, -8, 0, 0]],
    "RB_at_BR": [[0, 0, -12, 0, 0], [0, 16, 0, 16, 0], [-12, 0, 48, 0, -12], [0, 16, 0, 16, 0], [0, 0, -12, 0, 0]],
    "horizontal": [[0, 0, 4, 0, 0], [0, -8, 0, -8, 0], [-8, 32, 40, 32, -8], [0, -8, 0, -8, 0], [0, 0, 4, 0, 0]],
    "vertical": [[0, 0, -8, 0, 0], [0, -8, 32, -8, 0], [4, 0, 40, 0, 4], [0, -8, 32, -8, 0], [0, 0, -8, 0, 0]],
}


def _mhc_reference(img, x, y, pattern):
    """Demosaic pixel (x, y) by the textbook rule: the colour at a site is the raw value; a missing colour is
    the filter whose neighbours of that colour lie left/right ('horizontal') or above/below ('vertical') of a
    green site, the cross filter for green, the diagonal filter for the opposite colour. Integer arithmetic,
    division truncating toward zero, no clamping."""
    H, W = img.shape
    site = pattern[(y & 1) * 2 + (x & 1)]
    patch = np.array([[int(img[min(max(y - 2 + r, 0), H - 1), min(max(x - 2 + c, 0), W - 1)]) for c in range(5)] for r in range(5)])

    def filt(name):
        s = int((patch * np.array(MHC[name])).sum())
        return int(s / 64)  # truncation toward zero, like C++

    centre = int(patch[2, 2])
    if site == "R":
        return centre, filt("G_at_RB"), filt("RB_at_BR")
    if site == "B":
        return filt("RB_at_BR"), filt("G_at_RB"), centre
    # green: which colour shares this row?
    row_colour = pattern[(y & 1) * 2 + ((x + 1) & 1)]
    if row_colour == "R":
        return filt("horizontal"), centre, filt("vertical")
    return filt("vertical"), centre, filt("horizontal")


@pytest.mark.parametrize("code", ["GRBG", "RGGB", "GBRG", "BGGR"])
def test_bayer_against_the_published_filters(oracle, code):
    rng = np.random.default_rng(4)
    W, H = 24, 18
    img = rng.integers(0, 256, size=(H, W), dtype=np.uint8)
    pattern = list(code)
    for y in list(range(0, 6)) + [H - 2, H - 1]:
        for x in list(range(0, 6)) + [W - 2, W - 1]:
            want = np.array(_mhc_reference(img, x, y, pattern) + (255,), np.float32) * np.float32(1.0 / 255.0)
            got = oracle.fn_get_pixel(x, y, img, W, H, wl.fourcc(code))
            assert np.array_equal(got, want), (code, x, y)


def test_bayer_constant_mosaic_reproduces_itself(oracle):
    img = np.full((12, 16), 137, np.uint8)
    for code in ("GRBG", "RGGB", "GBRG", "BGGR"):
        got = oracle.fn_interpolate((5.3, 4.7), img, 16, 12, wl.fourcc(code))
        assert np.abs(got[:3] - 137 / 255.0).max() < 1e-6 and abs(got[3] - 1.0) < 1e-6


# ------------------------------------------------------------------ activations, dense, gather
def test_activations_against_float64(oracle):
    rng = np.random.default_rng(5)
    x = rng.normal(0, 2, (64, 5)).astype(np.float32)
    lam, alpha = 1.0507009873554804934193349852946, 1.6732632423543772848170429916717
    xd = x.astype(np.float64)
    assert np.abs(oracle.fn_activation(wl.SELU, x, 5) - np.where(xd >= 0, lam * xd, lam * (alpha * np.exp(xd) - alpha))).max() < 1e-6
    assert np.array_equal(oracle.fn_activation(wl.RELU, x, 5), np.maximum(x, 0))
    assert np.abs(oracle.fn_activation(wl.TANH, x, 5) - np.tanh(xd)).max() < 1e-6
    sm = oracle.fn_activation(wl.SOFTMAX, x, 5)
    assert np.abs(sm.sum(1) - 1).max() < 1e-6
    assert np.abs(sm - np.exp(xd) / np.exp(xd).sum(1, keepdims=True)).max() < 1e-6


def _small_case(oracle, net_groups, nn_model=wl.RING6):
    args = (nn_model, wl.SPHERE, 0.0949, 1.0, 2.0, 5.0) if nn_model == wl.RING6 else (nn_model, wl.CIRCLE, 0.05, 1.0, 3.0, 1.5)
    mesh = oracle.mesh(*args)
    lens = vmo.make_lens(160, 120, wl.EQUISOLID, 52.0, math.pi)
    Hoc = wl.make_hoc(1.0, math.radians(40), 0.05, 0.1)
    img = wl.random_image(np.random.default_rng(6), 160, 120, 4)
    feat = mesh.classify(Hoc, lens, img, wl.fourcc("RGBA"), vmo.Network([]))
    out = mesh.classify(Hoc, lens, img, wl.fourcc("RGBA"), vmo.Network(net_groups))
    return mesh, feat, out


def test_empty_network_returns_the_sampled_input_and_the_null_row(oracle):
    mesh, feat, _ = _small_case(oracle, [])
    V = len(feat["gidx"])
    assert V > 50 and feat["cls"].shape == (V + 1, 4)
    assert np.array_equal(feat["cls"][V], np.full(4, -1, np.float32))
    assert feat["cls"][:V].min() >= 0 and feat["cls"][:V].max() <= 1


def test_gather_order_is_self_then_neighbours_in_table_order(oracle):
    """A layer that copies input channel c of gather slot s to output s (identity-like weights, relu on
    non-negative data) exposes the gather order: out[i][s] = in[src(i, s)][c]."""
    nn = 6
    c = 1
    w = np.zeros(((nn + 1) * 4, nn + 1), np.float32)
    for s in range(nn + 1):
        w[s * 4 + c, s] = 1.0
    mesh, feat, out = _small_case(oracle, [[(w, np.zeros(nn + 1, np.float32), wl.RELU)]])
    V = len(out["gidx"])
    x = np.maximum(feat["cls"][:, c], 0)
    idx = np.concatenate([np.arange(V + 1)[:, None], out["nb"]], axis=1)
    assert np.array_equal(out["cls"], np.maximum(feat["cls"][:, c][idx], 0))
    assert x.shape[0] == V + 1


def test_network_against_float64_brute_force(oracle):
    rng = np.random.default_rng(8)
    groups = [
        [(rng.normal(0, 0.3, (28, 6)).astype(np.float32), rng.normal(0, 0.1, 6).astype(np.float32), wl.SELU),
         (rng.normal(0, 0.3, (6, 5)).astype(np.float32), rng.normal(0, 0.1, 5).astype(np.float32), wl.TANH)],
        [(rng.normal(0, 0.3, (35, 3)).astype(np.float32), rng.normal(0, 0.1, 3).astype(np.float32), wl.SOFTMAX)],
    ]
    mesh, feat, out = _small_case(oracle, groups)
    lam, alpha = 1.0507009873554804934193349852946, 1.6732632423543772848170429916717
    x = feat["cls"].astype(np.float64)
    N = x.shape[0]
    idx = np.concatenate([np.arange(N)[:, None], out["nb"]], axis=1)
    for group in groups:
        x = x[idx].reshape(N, -1)
        for (w, b, act) in group:
            y = x @ w.astype(np.float64) + b
            if act == wl.SELU:
                x = np.where(y >= 0, lam * y, lam * (alpha * np.exp(y) - alpha))
            elif act == wl.TANH:
                x = np.tanh(y)
            elif act == wl.RELU:
                x = np.maximum(y, 0)
            else:
                x = np.exp(y) / np.exp(y).sum(1, keepdims=True)
    assert np.abs(out["cls"] - x).max() < 2e-6


# ------------------------------------------------------------------ projection result invariants
@pytest.mark.parametrize("model", [wl.RING6, wl.NMGRID8])
def test_projected_mesh_invariants_and_brute_force_neighbourhood(oracle, model):
    args = (model, wl.SPHERE, 0.0949, 1.0, 3.0, 8.0) if model == wl.RING6 else (model, wl.CIRCLE, 0.05, 1.0, 4.0, 2.0)
    mesh = oracle.mesh(*args)
    rays, nbr = mesh.arrays()
    for name in sorted(LENSES):
        W, H, proj, f, fov = LENSES[name]
        lens = vmo.make_lens(W, H, proj, f / 4, fov)
        lens.width, lens.height = W // 4, H // 4
        Hoc = wl.make_hoc(1.0, math.radians(45), 0.1, 0.7)
        p = mesh.project(Hoc, lens)
        V = len(p["gidx"])
        assert V > 0
        assert np.all(np.diff(p["gidx"]) > 0), "global indices must be strictly ascending"
        assert np.all((p["px"][:, 0] >= 0) & (p["px"][:, 0] + 1 < lens.width) & (p["px"][:, 1] >= 0) & (p["px"][:, 1] + 1 < lens.height))
        # every kept node lies inside the lookup ranges, and its pixel is the projection of its own ray
        in_range = np.zeros(mesh.n_nodes, bool)
        for a, b in p["ranges"]:
            in_range[a:b] = True
        assert in_range[p["gidx"]].all()
        Rco = np.asarray(Hoc)[:3, :3].T
        for i in np.linspace(0, V - 1, 25).astype(int):
            cam = (Rco @ rays[p["gidx"][i]]).astype(np.float32)
            assert np.abs(oracle.fn_project(cam, lens) - p["px"][i]).max() < 1e-3
        # neighbourhood by brute force with a dictionary
        local = {int(g): i for i, g in enumerate(p["gidx"])}
        want = np.array([[local.get(int(n), V) for n in nbr[g]] for g in p["gidx"]] + [[V] * mesh.n_neighbours], np.int32)
        assert np.array_equal(p["nb"], want)


@pytest.mark.parametrize("model", [wl.RING6, wl.NMGRID8])
def test_lookup_graph_by_brute_force(oracle, model):
    """The LookupVisualMesh restatement against a dictionary walk in the other direction: every row starts with its own
    position; an entry >= 0 points at the row that holds exactly that neighbour; an entry < 0 is the most negative int32
    and its neighbour lies in no range (or is the null node); SAME edges differ from HARD edges only there, by the row's
    own position; the vectors are the rays of the range nodes in ascending order."""
    args = (model, wl.SPHERE, 0.0949, 1.0, 3.0, 8.0) if model == wl.RING6 else (model, wl.CIRCLE, 0.05, 1.0, 4.0, 2.0)
    mesh = oracle.mesh(*args)
    rays, nbr = mesh.arrays()
    W, H, proj, f, fov = LENSES["equisolid"]
    lens = vmo.make_lens(W // 4, H // 4, proj, f / 4, fov)
    Hoc = wl.make_hoc(1.0, math.radians(50), 0.1, 0.7)
    ranges = mesh.lookup(Hoc, lens)
    hard = mesh.lookup_graph(Hoc, lens)
    same = mesh.lookup_graph(Hoc, lens, same_edges=True)
    members = [g for a, b in ranges for g in range(a, b)]
    n = len(members)
    assert 0 < n < mesh.n_nodes, "the pose must cut the mesh for the edges to matter"
    assert hard["gidx"].tolist() == members and np.array_equal(hard["vectors"], rays[members])
    assert hard["graph"].shape == (n, mesh.n_neighbours + 1) and hard["graph"].dtype == np.int32
    position = {g: i for i, g in enumerate(members)}
    lowest = np.iinfo(np.int32).min
    missing = 0
    for i, g in enumerate(members):
        assert hard["graph"][i, 0] == i and same["graph"][i, 0] == i
        for j in range(mesh.n_neighbours):
            entry, neighbour = int(hard["graph"][i, j + 1]), int(nbr[g, j])
            if neighbour in position:
                assert entry == position[neighbour] and same["graph"][i, j + 1] == entry
            else:
                assert entry == lowest and same["graph"][i, j + 1] == i
                missing += 1
    assert missing > 0


def test_camera_looking_up_sees_nothing(oracle):
    mesh = oracle.mesh(wl.RING6, wl.SPHERE, 0.0949, 1.0, 3.0, 8.0)
    lens = vmo.make_lens(320, 256, wl.RECTILINEAR, 175.0, math.pi / 2)
    Hoc = wl.make_hoc(1.0, math.radians(-80), 0.0, 0.0)
    r = mesh.classify(Hoc, lens, np.zeros((256, 320 * 4), np.uint8), wl.fourcc("RGBA"), vmo.Network([]))
    assert len(r["gidx"]) == 0 and r["cls"].shape[0] == 0


# ------------------------------------------------------------------ mesh generation
def test_ring6_structure(oracle):
    r, h, k, d = 0.0949, 1.0, 3.0, 8.0
    mesh = oracle.mesh(wl.RING6, wl.SPHERE, r, h, k, d)
    rays, nbr = mesh.arrays()
    n = mesh.n_nodes
    assert np.abs(np.linalg.norm(rays, axis=1) - 1).max() < 1e-6
    # exactly one node straight down, all others point below the horizon and within max_distance
    down = np.flatnonzero((rays == np.array([0, 0, -1], np.float32)).all(1))
    assert len(down) == 1
    ground = h * np.sqrt(rays[:, 0] ** 2 + rays[:, 1] ** 2) / -rays[:, 2]
    assert ground.max() < d * 1.001
    # ring sizes: ceil(2 pi k / theta(n)) nodes on the ring n = i / k
    z_levels, counts = np.unique(np.round(rays[:, 2].astype(np.float64), 6), return_counts=True)
    order = np.argsort(z_levels)  # most negative z (closest ring) first
    ring_counts = counts[order][1:6]
    want = [math.ceil(2 * math.pi * k / oracle.fn_shape(wl.SPHERE, r, "theta", i / k, h)) for i in range(1, 6)]
    assert ring_counts.tolist() == want
    # neighbour indices are valid and the left/right links (slots 0 and 3) are mutual
    assert nbr.min() >= 0 and nbr.max() <= n
    for i in range(1, n, max(1, n // 300)):
        left, right = nbr[i, 0], nbr[i, 3]
        if left < n and left != 0 and i != int(down[0]):
            assert nbr[left, 3] == i
        if right < n and right != 0 and i != int(down[0]):
            assert nbr[right, 0] == i


def test_nmgrid8_structure(oracle):
    mesh = oracle.mesh(wl.NMGRID8, wl.CIRCLE, 0.05, 1.0, 4.0, 2.0)
    rays, nbr = mesh.arrays()
    n = mesh.n_nodes
    assert np.abs(np.linalg.norm(rays, axis=1) - 1).max() < 1e-6
    ground = np.sqrt(rays[:, 0] ** 2 + rays[:, 1] ** 2) / -rays[:, 2]
    assert ground.max() <= 2.0 * 1.001
    # 8-neighbour grid: opposite slots are mutual (0 left <-> 4 right, 2 top <-> 6 bottom, diagonals 1<->5, 3<->7)
    for i in range(0, n, max(1, n // 400)):
        for s in range(8):
            j = nbr[i, s]
            if j < n:
                assert nbr[j, (s + 4) % 8] == i
    # for a flat circle the n-th object along x sits at x = 2 r n: the node spacing along the axes is 2r/k
    axis = rays[(np.abs(rays[:, 1]) < 1e-7) & (rays[:, 0] > 0)]
    xs = np.sort(axis[:, 0] / -axis[:, 2])
    assert np.abs(np.diff(xs) - 2 * 0.05 / 4.0).max() < 1e-4


def test_sphere_n_inverts_phi(oracle):
    for n in (0.7, 2.0, 11.5, 40.0):
        phi = oracle.fn_shape(wl.SPHERE, 0.0949, "phi", n, 1.2)
        assert abs(oracle.fn_shape(wl.SPHERE, 0.0949, "n", phi, 1.2) - n) < 2e-3 * max(1, n)
    # closed form: phi(n) = atan(sinh(-n ln(1 - 2r/h)))
    assert abs(oracle.fn_shape(wl.SPHERE, 0.1, "phi", 3.0, 1.0) - math.atan(math.sinh(-3.0 * math.log(1 - 0.2)))) < 1e-6
    assert abs(oracle.fn_shape(wl.CIRCLE, 0.05, "phi", 3.0, 1.0) - math.atan(0.3)) < 1e-6

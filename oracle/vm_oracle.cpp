/*
 * vm_oracle.cpp - CPU restatement of the reference Visual Mesh inference path for one Scalar type:
 * `real` is float (libvm_oracle.so) or, compiled with -DVMO_REAL=double, double (libvm_oracle_f64.so).
 *
 * TEST INFRASTRUCTURE ONLY: the checker for the HIP engine and the timed CPU baseline. The shipped
 * engine never links or loads this file.
 *
 * Every function names the reference file:line it follows (paths relative to the reference's
 * cpp/visualmesh/). The arithmetic is written out with the exact operand types and evaluation order
 * the reference's templates have for Scalar=real (where the reference mixes a double literal into a
 * Scalar expression the promotion to double and the rounding back are spelled out; for real=double
 * they change nothing), because the node order, the lookup ranges and the visible set all hang on
 * last-bit comparisons. Build with -O2 -ffp-contract=off, no -march=native, no -ffast-math (see
 * Makefile), so that every operation on reals is a single IEEE-754 operation of that type.
 *
 * Parity status: every function here is pinned bit-for-bit against the compiled reference headers
 * (_ref/libvm_ref.so, tests/test_oracle_vs_reference.py) wherever the reference tree is mounted, and
 * against closed forms / invariants / committed golden vectors everywhere else (tests/test_oracle_*.py).
 * The one thing only the differential run can pin is the exact BSP permutation and the heuristic
 * lookup ranges; the golden digests under tests/golden/ were written from a run in which the
 * differential test passed.
 */
#include "vm_oracle.h"

#include <algorithm>
#include <array>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <limits>
#include <map>
#include <numeric>
#include <set>
#include <stdexcept>
#include <utility>
#include <vector>

typedef vmo_real real;

namespace {

typedef std::array<real, 3> V3;
typedef std::array<real, 2> V2;

/* utility/math.hpp:145-164: dot is the recursion a[L-1]*b[L-1] + dot_{L-2}, i.e. for three
 * components a2*b2 + (a1*b1 + a0*b0). */
inline real dot3(const V3& a, const V3& b) { return a[2] * b[2] + (a[1] * b[1] + a[0] * b[0]); }
inline real dot2(const V2& a, const V2& b) { return a[1] * b[1] + a[0] * b[0]; }
/* utility/math.hpp:166-175 */
inline real norm3(const V3& a) { return std::sqrt(dot3(a, a)); }
inline V3 normalise3(const V3& a) {
    const real len = real(1.0) / norm3(a);
    return V3{{a[0] * len, a[1] * len, a[2] * len}};
}
/* utility/math.hpp:177-184 */
inline V3 cross3(const V3& a, const V3& b) {
    return V3{{a[1] * b[2] - a[2] * b[1], a[2] * b[0] - a[0] * b[2], a[0] * b[1] - a[1] * b[0]}};
}
struct M3 {
    V3 r[3];
};
/* utility/math.hpp:254-257 */
inline V3 mul(const M3& m, const V3& v) { return V3{{dot3(m.r[0], v), dot3(m.r[1], v), dot3(m.r[2], v)}}; }

/* Rco = block<3,3>(transpose(Hoc)) : engine/cpu/engine.hpp:95, mesh.hpp:507 */
inline M3 rco_from_hoc(const real* H) {
    M3 m;
    for (int i = 0; i < 3; ++i)
        for (int j = 0; j < 3; ++j) m.r[i][j] = H[j * 4 + i];
    return m;
}

/* ------------------------------------------------------------------ shapes */
struct Shape {
    int kind;
    real r;
    /* geometry/Sphere.hpp:66-68, geometry/Circle.hpp:72-74 */
    real phi(real n, real h) const {
        if (kind == VMO_SHAPE_SPHERE) return -std::atan(std::sinh(n * std::log1p(-real(2.0) * r / h)));
        return std::atan((real(2.0) * n * r) / h);
    }
    /* geometry/Sphere.hpp:80-82, geometry/Circle.hpp:85-87 */
    real n(real phi_, real h) const {
        if (kind == VMO_SHAPE_SPHERE) return std::asinh(std::tan(-phi_)) / std::log1p(-real(2.0) * r / h);
        return (h * std::tan(phi_)) / (real(2.0) * r);
    }
    /* geometry/Sphere.hpp:97-99, geometry/Circle.hpp:101-103 */
    real k(real h0, real h1) const {
        if (kind == VMO_SHAPE_SPHERE)
            return (std::log(h1 - 2 * r) - std::log(h1)) / (std::log(h0 - 2 * r) - std::log(h0));
        return h0 / h1;
    }
    /* geometry/Sphere.hpp:106-108, geometry/Circle.hpp:110-112 */
    real c() const { return kind == VMO_SHAPE_SPHERE ? r : real(0.0); }
    /* geometry/Sphere.hpp:124-130, geometry/Circle.hpp:128-134. The first arm divides in double
     * (the literal 1.0), the conditional's common type is double, the return rounds to real. */
    real theta(real n, real h) const {
        const double v = n <= 0.5 ? double(real(2.0 * M_PI)) / (1.0 + double(n * real(2.0)))
                                  : double(real(2.0) * std::asin(r / ((h - r) * std::tan(phi(n, h)))));
        return real(v);
    }
};

/* ------------------------------------------------------------------ lens maths */
/* utility/projection.hpp:104-120: the literal 1.0 makes the bracket a double sum of real terms. */
inline real distort(real r, const real* k) {
    const real ik0 = -k[0];
    const real ik1 = real(3.0) * (k[0] * k[0]) - k[1];
    const real ik2 = -real(12.0) * (k[0] * k[0]) * k[0] + real(8.0) * k[0] * k[1];
    const real ik3 = real(55.0) * (k[0] * k[0]) * (k[0] * k[0]) - real(55.0) * (k[0] * k[0]) * k[1] + real(5.0) * (k[1] * k[1]);
    const double s = 1.0 + double(ik0 * (r * r)) + double(ik1 * ((r * r) * (r * r)))
                     + double(ik2 * ((r * r) * (r * r)) * (r * r))
                     + double(ik3 * ((r * r) * (r * r)) * ((r * r) * (r * r)));
    return real(double(r) * s);
}
/* utility/projection.hpp:138-144 */
inline real undistort(real r, const real* k) {
    return real(double(r) * (1.0 + double(k[0] * (r * r)) + double(k[1] * ((r * r) * (r * r)))));
}

/* utility/projection.hpp:162-187 */
inline V2 project(const V3& ray, const vmo_lens& lens) {
    const real f = lens.focal_length;
    const real theta = std::acos(ray[0]);
    const real rsin_theta = real(1.0) / std::sqrt(real(1.0) - ray[0] * ray[0]);
    real r_u;
    switch (lens.projection) {
        case VMO_RECTILINEAR: r_u = f * std::tan(std::min(std::max(theta, real(0.0)), real(M_PI_2))); break;
        case VMO_EQUISOLID: r_u = real(2.0) * f * std::sin(theta * real(0.5)); break;
        case VMO_EQUIDISTANT: r_u = f * theta; break;
        default: throw std::runtime_error("Cannot project: Unknown lens type");
    }
    const real r_d = distort(r_u, lens.k);
    V2 screen = ray[0] >= 1 ? V2{{real(0.0), real(0.0)}} : V2{{r_d * ray[1] * rsin_theta, r_d * ray[2] * rsin_theta}};
    const real cx = real(lens.width) * real(0.5), cy = real(lens.height) * real(0.5);
    return V2{{(cx - screen[0]) - lens.centre[0], (cy - screen[1]) - lens.centre[1]}};
}

/* utility/projection.hpp:204-225 */
inline V3 unproject(const V2& px, const vmo_lens& lens) {
    const V2 screen{{real(lens.width) * real(0.5) - (px[0] + lens.centre[0]),
                     real(lens.height) * real(0.5) - (px[1] + lens.centre[1])}};
    const real f = lens.focal_length;
    const real r_d = std::sqrt(dot2(screen, screen));
    if (r_d == 0) return V3{{real(1.0), real(0.0), real(0.0)}};
    const real r_u = undistort(r_d, lens.k);
    real theta;
    switch (lens.projection) {
        case VMO_RECTILINEAR: theta = std::atan(r_u / f); break;
        case VMO_EQUISOLID: theta = real(2.0) * std::asin(r_u / (real(2.0) * f)); break;
        case VMO_EQUIDISTANT: theta = r_u / f; break;
        default: throw std::runtime_error("Cannot project: Unknown lens type");
    }
    const real sin_theta = std::sin(theta);
    return V3{{std::cos(theta), sin_theta * screen[0] / r_d, sin_theta * screen[1] / r_d}};
}

/* ------------------------------------------------------------------ cones */
struct Cone {
    V3 axis;
    real cos_t;
};
/* utility/cone.hpp:32-34, :46-48, :61-66, :80-98 */
inline Cone cone0() { return Cone{V3{{0, 0, 0}}, 1}; }
inline Cone cone1(const V3& p1) { return Cone{p1, 1}; }
inline Cone cone2(const V3& p1, const V3& p2) {
    const V3 axis = normalise3(V3{{p1[0] + p2[0], p1[1] + p2[1], p1[2] + p2[2]}});
    return Cone{axis, dot3(axis, p1)};
}
inline Cone cone3(const V3& p1, const V3& p2, const V3& p3) {
    /* invert(): utility/math.hpp:275-301 */
    const V3 m[3] = {p1, p2, p3};
    const real det = (m[0][0] * (m[1][1] * m[2][2] - m[2][1] * m[1][2]) - m[0][1] * (m[1][0] * m[2][2] - m[1][2] * m[2][0])
                       + m[0][2] * (m[1][0] * m[2][1] - m[1][1] * m[2][0]));
    V3 im[3];
    if (det == 0) {
        const real nan = std::numeric_limits<real>::quiet_NaN();
        im[0] = im[1] = im[2] = V3{{nan, nan, nan}};
    }
    else {
        const real idet = real(1.0) / det;
        im[0] = V3{{(m[1][1] * m[2][2] - m[2][1] * m[1][2]) * idet, (m[0][2] * m[2][1] - m[0][1] * m[2][2]) * idet,
                    (m[0][1] * m[1][2] - m[0][2] * m[1][1]) * idet}};
        im[1] = V3{{(m[1][2] * m[2][0] - m[1][0] * m[2][2]) * idet, (m[0][0] * m[2][2] - m[0][2] * m[2][0]) * idet,
                    (m[1][0] * m[0][2] - m[0][0] * m[1][2]) * idet}};
        im[2] = V3{{(m[1][0] * m[2][1] - m[2][0] * m[1][1]) * idet, (m[2][0] * m[0][1] - m[0][0] * m[2][1]) * idet,
                    (m[0][0] * m[1][1] - m[1][0] * m[0][1]) * idet}};
    }
    const V3 ones{{1, 1, 1}};
    const V3 axis = normalise3(V3{{dot3(im[0], ones), dot3(im[1], ones), dot3(im[2], ones)}});
    return Cone{axis, dot3(axis, p1)};
}

struct BspCone {
    V3 axis;
    real cos_t, sin_t;
};

}  // namespace

/* ------------------------------------------------------------------ mesh */
struct vmo_mesh {
    int nn = 0;
    real h = 0, max_distance = 0;
    std::vector<V3> rays;
    std::vector<int> nbr; /* [n][nn], global indices, n_nodes means "no neighbour" */
    struct Bsp {
        int first, second;
        int child[2];
        BspCone cone;
    };
    std::vector<Bsp> bsp;
    int n() const { return int(rays.size()); }
};

namespace {

/* model/polar_map.hpp:41-43, :56-72 */
V3 polar_map(const Shape& s, real h, real n, real m) {
    const real phi = s.phi(std::abs(n), h);
    const real d_theta = s.theta(std::abs(n), h);
    const real theta = real(double(d_theta * m) + (n < 0 ? M_PI : 0.0));
    return V3{{std::cos(theta) * std::sin(phi), std::sin(theta) * std::sin(phi), -std::cos(phi)}};
}

/* model/ring6.hpp:50-69 */
std::array<int, 6> ring6_neighbours(int i, int p, int c, int n) {
    const real f = real(i) / real(c);
    const int l = i > 0 ? i - 1 : c - 1;
    const int r = i + 1 < c ? i + 1 : 0;
    const int tl = (int(f * n) % n) + c;
    const int tr = ((int(f * n) + 1) % n) + c;
    const int bl = (int(f * p) % p) - p;
    const int br = ((int(f * p) + 1) % p) - p;
    return std::array<int, 6>{{l, tl, tr, r, br, bl}};
}

/* model/ring_base.hpp:53-115 with Ring = Ring6 */
void generate_ring6(vmo_mesh& mesh, const Shape& shape, real h, real k, real max_distance) {
    const int N = 6;
    mesh.nn = N;
    const real jump = real(1.0 / double(k));
    const real two_pi = real(2.0 * M_PI);
    int start = 1;

    mesh.rays.push_back(V3{{real(0.0), real(0.0), -real(1.0)}});
    mesh.nbr.resize(N, 0);
    const int n_first = int(std::ceil((k * two_pi) / shape.theta(jump, h)));
    const real first_jump = real(n_first) / real(N);
    for (unsigned int i = 0; i < unsigned(N); ++i) mesh.nbr[i] = int(i * first_jump) + start;

    for (int i = 1; h * std::tan(shape.phi(i * jump, h)) < max_distance; ++i) {
        const real n_p = (i - 1) * jump;
        const real n_c = i * jump;
        const real n_n = (i + 1) * jump;

        const real s_p = i == 1 ? real(1.0) : k * two_pi / shape.theta(n_p, h);
        const real s_c = k * two_pi / shape.theta(n_c, h);
        const real s_n = k * two_pi / shape.theta(n_n, h);

        const real m_jump = s_c / (k * std::ceil(s_c));

        start = int(mesh.rays.size());
        const int ip = int(std::ceil(s_p)), ic = int(std::ceil(s_c)), in = int(std::ceil(s_n));
        for (int j = 0; j < ic; ++j) {
            mesh.rays.push_back(polar_map(shape, h, n_c, j * m_jump));
            const std::array<int, 6> rel = ring6_neighbours(j, ip, ic, in);
            for (int t = 0; t < N; ++t) mesh.nbr.push_back(start + rel[t]);
        }
    }
    const int total = int(mesh.rays.size());
    for (int i = start - 1; i < total; ++i)
        for (int t = 0; t < N; ++t) mesh.nbr[size_t(i) * N + t] = std::min(mesh.nbr[size_t(i) * N + t], total);
}

/* model/nmgrid_map.hpp:33-64 */
V3 nm_xyz(const Shape& s, real h, real n, real h_n) {
    const real c = s.c();
    const real x = (h_n - c) * std::tan(s.phi(n, h_n));
    const real y = std::sqrt((h_n - c) * (h_n - c) - (h - c) * (h - c));
    return V3{{x, y, c - h}};
}
real nm_guess_m(const Shape& s, real h, real n, real h_n) {
    const real c = s.c();
    const V3 v = nm_xyz(s, h, n, h_n);
    const real h_m = std::sqrt(v[0] * v[0] + v[2] * v[2]) + c;
    const real phi_m = std::acos(std::sqrt((v[0] * v[0] + v[2] * v[2]) / (v[0] * v[0] + v[1] * v[1] + v[2] * v[2])));
    return s.n(phi_m, h_m);
}
/* model/nmgrid_map.hpp:95-131: bisection on the plane height of the first coordinate */
V3 nmgrid_map(const Shape& s, real h, real nm0, real nm1) {
    const real n = std::abs(nm0);
    const real m = std::abs(nm1);
    const real c = s.c();
    real lo = h;
    real hi = (h - c) / std::cos(s.phi(m, h)) + c;
    real h_n = real(double(lo + hi) * 0.5);
    while (true) {
        if (h_n == lo || h_n == hi) break;
        const real m_g = nm_guess_m(s, h, n, h_n);
        (m_g > m ? hi : lo) = h_n;
        if (double(h_n) == double(lo + hi) * 0.5) break;
        h_n = real(double(lo + hi) * 0.5);
    }
    V3 v = nm_xyz(s, h, n, h_n);
    v[0] *= nm0 >= 0 ? 1 : -1;
    v[1] *= nm1 >= 0 ? 1 : -1;
    return v;
}

/* model/grid_base.hpp:78-144 with Map = NMGridMap, 8 neighbours. The flood fill order (LIFO stack,
 * offsets in the table's order) fixes the node order; the containers only answer membership. */
void generate_nmgrid8(vmo_mesh& mesh, const Shape& shape, real h, real k, real max_distance) {
    const int N = 8;
    mesh.nn = N;
    static const int off[8][2] = {{-1, 0}, {-1, 1}, {0, 1}, {1, 1}, {1, 0}, {1, -1}, {0, -1}, {-1, -1}};
    const real jump = real(1.0 / double(k));
    typedef std::pair<int, int> C2;
    std::map<C2, int> locations;
    std::set<C2> seen;
    std::vector<C2> stack;
    seen.insert(C2(0, 0));
    stack.push_back(C2(0, 0));
    while (!stack.empty()) {
        const C2 e = stack.back();
        stack.pop_back();
        const real nm0 = real(e.first) * jump, nm1 = real(e.second) * jump;
        const V3 vec = nmgrid_map(shape, h, nm0, nm1);
        const real distance = std::sqrt(dot2(V2{{vec[0], vec[1]}}, V2{{vec[0], vec[1]}}));
        if (distance <= max_distance) {
            locations.emplace(e, int(mesh.rays.size()));
            mesh.rays.push_back(normalise3(vec));
            for (int t = 0; t < N; ++t) {
                const C2 nb(e.first + off[t][0], e.second + off[t][1]);
                if (seen.count(nb) == 0) {
                    seen.insert(nb);
                    stack.push_back(nb);
                }
            }
        }
    }
    const int total = int(mesh.rays.size());
    mesh.nbr.assign(size_t(total) * N, total);
    for (const auto& loc : locations) {
        for (int t = 0; t < N; ++t) {
            auto it = locations.find(C2(loc.first.first + off[t][0], loc.first.second + off[t][1]));
            mesh.nbr[size_t(loc.second) * N + t] = it != locations.end() ? it->second : total;
        }
    }
}

/* mesh.hpp:96-118: incremental smallest bounding cone over the index order given */
typedef std::vector<int>::iterator It;
BspCone bounding_cone(const vmo_mesh& mesh, It start, It end) {
    const std::vector<V3>& R = mesh.rays;
    Cone cone = cone0();
    for (It i = start; i < end; ++i) {
        if (dot3(cone.axis, R[*i]) < cone.cos_t) {
            cone = cone1(R[*i]);
            for (It j = start; j < i; ++j) {
                if (dot3(cone.axis, R[*j]) < cone.cos_t) {
                    cone = cone2(R[*i], R[*j]);
                    for (It k = start; k < j; ++k) {
                        if (dot3(cone.axis, R[*k]) < cone.cos_t) cone = cone3(R[*i], R[*j], R[*k]);
                    }
                }
            }
        }
    }
    return BspCone{cone.axis, cone.cos_t, std::sqrt(real(1.0) - cone.cos_t * cone.cos_t)};
}

/* mesh.hpp:135-248. std::partition / std::sort / std::max_element on std::vector<int>::iterator, as in
 * the reference, so the resulting permutation is the same one. */
int build_bsp(vmo_mesh& mesh, It start, It end, int min_points, int offset) {
    const std::vector<V3>& R = mesh.rays;
    const int count = int(std::distance(start, end));
    if (count == 0) throw std::runtime_error("We tried to make a tree with no nodes");

    if (count <= min_points) {
        const int elem = int(mesh.bsp.size());
        mesh.bsp.push_back(vmo_mesh::Bsp{offset, offset + count, {-1, -1}, bounding_cone(mesh, start, end)});
        std::sort(start, end);
        return elem;
    }

    if (mesh.bsp.empty()) {
        It max_phi_element = std::max_element(start, end, [&R](const int& a, const int& b) { return R[a][2] < R[b][2]; });
        const real cone_cos = -R[*max_phi_element][2];
        const real cone_sin = std::sqrt(1 - cone_cos * cone_cos);
        It mid = std::partition(start, end, [&R](const int& a) { return R[a][1] > 0; });
        mesh.bsp.push_back(vmo_mesh::Bsp{offset, count, {-1, -1}, BspCone{V3{{0, 0, -1}}, cone_cos, cone_sin}});
        const int c0 = build_bsp(mesh, start, mid, min_points, 0);
        const int c1 = build_bsp(mesh, mid, end, min_points, int(std::distance(start, mid)));
        mesh.bsp.front().child[0] = c0;
        mesh.bsp.front().child[1] = c1;
        return 0;
    }

    const BspCone cone = bounding_cone(mesh, start, end);

    real min_phi = std::numeric_limits<real>::max();
    real max_phi = std::numeric_limits<real>::lowest();
    real min_theta = std::numeric_limits<real>::max();
    real max_theta = std::numeric_limits<real>::lowest();
    real sum_theta = 0, sum_phi = 0;
    int count_theta = 0, count_phi = 0;
    for (It it = start; it != end; ++it) {
        const V3& ray = R[*it];
        const real phi = ray[2];
        const real theta = ray[0] / std::sqrt(1 - ray[2] * ray[2]);
        min_phi = std::min(min_phi, phi);
        max_phi = std::max(max_phi, phi);
        sum_phi += phi;
        count_phi += 1;
        if (std::isfinite(theta)) {
            min_theta = std::min(min_theta, theta);
            max_theta = std::max(max_theta, theta);
            sum_theta += theta;
            count_theta += 1;
        }
    }
    const real split_phi = sum_phi / count_phi;
    const real split_theta = sum_theta / count_theta;

    It mid = max_phi - min_phi > max_theta - min_theta
               ? std::partition(start, end, [&R, &split_phi](const int& a) { return R[a][2] > split_phi; })
               : std::partition(start, end, [&R, &split_theta](const int& a) {
                     return R[a][0] / std::sqrt(1 - R[a][2] * R[a][2]) < split_theta;
                 });

    const int elem = int(mesh.bsp.size());
    mesh.bsp.push_back(vmo_mesh::Bsp{offset, offset + count, {-1, -1}, cone});
    const int c0 = build_bsp(mesh, start, mid, min_points, offset);
    const int c1 = build_bsp(mesh, mid, end, min_points, offset + int(std::distance(start, mid)));
    mesh.bsp[elem].child[0] = c0;
    mesh.bsp[elem].child[1] = c1;
    return elem;
}

/* mesh.hpp:424-467 */
void finish_mesh(vmo_mesh& mesh) {
    const int n = mesh.n();
    const int nn = mesh.nn;
    std::vector<int> sorting(n);
    std::iota(sorting.begin(), sorting.end(), 0);
    uint32_t x = 0x4d657368;
    for (int i = n - 1; i > 0; i -= 5) {
        x ^= x << 13;
        x ^= x >> 17;
        x ^= x << 5;
        std::swap(sorting[i], sorting[x % i]);
    }
    mesh.bsp.reserve(size_t(n) * 2);
    build_bsp(mesh, sorting.begin(), sorting.end(), 8, 0);

    std::vector<int> r_sorting(size_t(n) + 1);
    r_sorting[n] = n;
    for (int i = 0; i < n; ++i) r_sorting[sorting[i]] = i;

    std::vector<V3> rays(n);
    std::vector<int> nbr(size_t(n) * nn);
    for (int i = 0; i < n; ++i) {
        rays[i] = mesh.rays[sorting[i]];
        for (int t = 0; t < nn; ++t) nbr[size_t(i) * nn + t] = r_sorting[mesh.nbr[size_t(sorting[i]) * nn + t]];
    }
    mesh.rays.swap(rays);
    mesh.nbr.swap(nbr);
}

/* mesh.hpp:265-349 */
void screen_edges(const real* H, const vmo_lens& lens, BspCone edges[4]) {
    M3 Roc;
    for (int i = 0; i < 3; ++i)
        for (int j = 0; j < 3; ++j) Roc.r[i][j] = H[i * 4 + j];
    const V2 dims{{real(lens.width) - real(1.0), real(lens.height) - real(1.0)}};
    const V3 rN[4] = {
      mul(Roc, unproject(V2{{1, 1}}, lens)),
      mul(Roc, unproject(V2{{dims[0], 1}}, lens)),
      mul(Roc, unproject(V2{{dims[0], dims[1]}}, lens)),
      mul(Roc, unproject(V2{{1, dims[1]}}, lens)),
    };
    switch (lens.projection) {
        case VMO_RECTILINEAR: {
            edges[0] = BspCone{normalise3(cross3(rN[1], rN[0])), 0, 1};
            edges[1] = BspCone{normalise3(cross3(rN[2], rN[1])), 0, 1};
            edges[2] = BspCone{normalise3(cross3(rN[3], rN[2])), 0, 1};
            edges[3] = BspCone{normalise3(cross3(rN[0], rN[3])), 0, 1};
            return;
        }
        case VMO_EQUIDISTANT:
        case VMO_EQUISOLID: {
            const V2 centre{{dims[0] * real(0.5) + lens.centre[0], dims[1] * real(0.5) + lens.centre[1]}};
            const V3 rE[4] = {
              mul(Roc, unproject(V2{{centre[0], 1}}, lens)),
              mul(Roc, unproject(V2{{dims[0], centre[1]}}, lens)),
              mul(Roc, unproject(V2{{centre[0], dims[1]}}, lens)),
              mul(Roc, unproject(V2{{1, centre[1]}}, lens)),
            };
            const Cone c[4] = {cone3(rN[1], rE[0], rN[0]), cone3(rN[2], rE[1], rN[1]), cone3(rN[3], rE[2], rN[2]),
                               cone3(rN[0], rE[3], rN[3])};
            for (int i = 0; i < 4; ++i) edges[i] = BspCone{c[i].axis, c[i].cos_t, std::sqrt(real(1.0) - c[i].cos_t * c[i].cos_t)};
            return;
        }
        default: throw std::runtime_error("Unknown lens type");
    }
}

/* mesh.hpp:362-406 */
std::pair<bool, bool> check_on_screen(const M3& Rco, const BspCone& cone, const vmo_lens& lens, const BspCone edges[4]) {
    const V2 px = project(mul(Rco, cone.axis), lens);
    const bool axis_on_screen = 0 <= px[0] && px[0] + 1 <= lens.width && 0 <= px[1] && px[1] + 1 <= lens.height;
    real angles[4];
    bool contains[4];
    for (int i = 0; i < 4; ++i) {
        angles[i] = dot3(cone.axis, edges[i].axis);
        contains[i] = angles[i] > edges[i].cos_t * cone.cos_t + edges[i].sin_t * cone.sin_t;
    }
    const bool outside = !axis_on_screen && (contains[0] || contains[1] || contains[2] || contains[3]);
    if (outside) return std::make_pair(false, true);
    bool intersects[4];
    for (int i = 0; i < 4; ++i) intersects[i] = angles[i] < edges[i].cos_t * cone.cos_t - edges[i].sin_t * cone.sin_t;
    const bool inside = axis_on_screen && intersects[0] && intersects[1] && intersects[2] && intersects[3];
    return std::make_pair(inside, outside);
}

/* mesh.hpp:499-595 */
std::vector<std::pair<int, int>> lookup(const vmo_mesh& mesh, const real* H, const vmo_lens& lens) {
    const real cos_fov = std::cos(lens.fov * real(0.5));
    const real sin_fov = std::sin(lens.fov * real(0.5));
    const M3 Rco = rco_from_hoc(H);
    const V3 rXCo = Rco.r[0];
    BspCone edges[4];
    screen_edges(H, lens, edges);

    std::vector<int> stack(1, 0);
    std::vector<std::pair<int, int>> ranges;
    bool building = false;
    int range_start = 0, range_end = 0;
    while (!stack.empty()) {
        const int i = stack.back();
        stack.pop_back();
        const vmo_mesh::Bsp& elem = mesh.bsp[i];
        const BspCone& cone = elem.cone;

        const real delta = dot3(rXCo, cone.axis);
        bool outside = delta < cos_fov * cone.cos_t - sin_fov * cone.sin_t;
        bool inside = delta > cos_fov * cone.cos_t + sin_fov * cone.sin_t;
        if (!outside && inside) {
            const std::pair<bool, bool> io = check_on_screen(Rco, cone, lens, edges);
            inside = io.first;
            outside = io.second;
        }

        if (inside) {
            if (building) { range_end = elem.second; }
            else {
                range_start = elem.first;
                range_end = elem.second;
                building = true;
            }
        }
        else if (outside) {
            if (building) {
                ranges.emplace_back(range_start, range_end);
                building = false;
            }
        }
        else if (elem.child[0] < 0) {
            for (int j = elem.first; j < elem.second; ++j) {
                const V2 px = project(mul(Rco, mesh.rays[j]), lens);
                const bool on_screen = dot3(rXCo, mesh.rays[j]) > cos_fov && 0 <= px[0] && px[0] + 1 <= lens.width
                                       && 0 <= px[1] && px[1] + 1 <= lens.height;
                if (on_screen && building) { range_end = j + 1; }
                else if (!on_screen && building) {
                    ranges.emplace_back(range_start, range_end);
                    building = false;
                }
                else if (on_screen && !building) {
                    range_start = j;
                    range_end = j + 1;
                    building = true;
                }
            }
        }
        else {
            stack.push_back(elem.child[1]);
            stack.push_back(elem.child[0]);
        }
    }
    if (building) ranges.emplace_back(range_start, range_end);
    return ranges;
}

/* ------------------------------------------------------------------ image sampling */
inline uint32_t cc(const char (&c)[5]) { return uint32_t(c[0] | (c[1] << 8) | (c[2] << 16) | (c[3] << 24)); }

/* engine/cpu/bayer.hpp:45-79: Malvar-He-Cutler kernels scaled by 64 */
const int G_R[25] = {0, 0, -8, 0, 0, 0, 0, 16, 0, 0, -8, 16, 32, 16, -8, 0, 0, 16, 0, 0, 0, 0, -8, 0, 0};
const int R_B[25] = {0, 0, -12, 0, 0, 0, 16, 0, 16, 0, -12, 0, 48, 0, -12, 0, 16, 0, 16, 0, 0, 0, -12, 0, 0};
const int R_GR[25] = {0, 0, 4, 0, 0, 0, -8, 0, -8, 0, -8, 32, 40, 32, -8, 0, -8, 0, -8, 0, 0, 0, 4, 0, 0};
const int R_GB[25] = {0, 0, -8, 0, 0, 0, -8, 32, -8, 0, 4, 0, 40, 0, 4, 0, -8, 32, -8, 0, 0, 0, -8, 0, 0};
const int* const G_B = G_R;
const int* const B_R = R_B;
const int* const B_GB = R_GR;
const int* const B_GR = R_GB;
enum BayerType { BT_R, BT_GR, BT_GB, BT_B };

inline int idot25(const int* p, const int* k) {
    int s = 0;
    for (int i = 0; i < 25; ++i) s += p[i] * k[i];
    return s;
}

/* engine/cpu/bayer.hpp:95-108: integer dot, C++ truncating division by 64, no clamp, alpha 255 */
void demosaic(const int* p, BayerType type, real* out) {
    int o[4];
    switch (type) {
        case BT_R: o[0] = p[12], o[1] = idot25(p, G_R) / 64, o[2] = idot25(p, B_R) / 64; break;
        case BT_GR: o[0] = idot25(p, R_GR) / 64, o[1] = p[12], o[2] = idot25(p, B_GR) / 64; break;
        case BT_GB: o[0] = idot25(p, R_GB) / 64, o[1] = p[12], o[2] = idot25(p, B_GB) / 64; break;
        default: o[0] = idot25(p, R_B) / 64, o[1] = idot25(p, G_B) / 64, o[2] = p[12]; break;
    }
    o[3] = 255;
    const real s = real(1.0 / 255.0);
    for (int i = 0; i < 4; ++i) out[i] = real(o[i]) * s;
}

/* engine/cpu/bayer.hpp:122-158 */
int bayer_get_pixel(int px, int py, const uint8_t* image, int W, int H, uint32_t format, real* out) {
    int patch[25];
    for (int y = 0; y < 5; ++y) {
        const int yc = std::min(std::max(py - 2 + y, 0), H - 1);
        for (int x = 0; x < 5; ++x) {
            const int xc = std::min(std::max(px - 2 + x, 0), W - 1);
            patch[y * 5 + x] = image[yc * W + xc];
        }
    }
    const bool col = px % 2 == 1;
    const bool row = py % 2 == 1;
    BayerType t;
    if (format == cc("GRBG")) t = row ? (col ? BT_GB : BT_B) : (col ? BT_R : BT_GR);
    else if (format == cc("RGGB")) t = row ? (col ? BT_B : BT_GB) : (col ? BT_GR : BT_R);
    else if (format == cc("GBRG")) t = row ? (col ? BT_GR : BT_R) : (col ? BT_B : BT_GB);
    else if (format == cc("BGGR")) t = row ? (col ? BT_R : BT_GR) : (col ? BT_GB : BT_B);
    else return VMO_ERR_FORMAT;
    demosaic(patch, t, out);
    return VMO_OK;
}

/* engine/cpu/pixel.hpp:43-102 */
int get_pixel(int x, int y, const uint8_t* im, int W, int H, uint32_t format, real* o) {
    const real s = real(1.0 / 255.0);
    if (format == cc("GRBG") || format == cc("RGGB") || format == cc("GBRG") || format == cc("BGGR"))
        return bayer_get_pixel(x, y, im, W, H, format, o);
    if (format == cc("BGR3") || format == cc("BGR8")) {
        const int c = (y * W + x) * 3;
        o[0] = im[c + 2] * s, o[1] = im[c + 1] * s, o[2] = im[c + 0] * s, o[3] = real(1.0);
        return VMO_OK;
    }
    if (format == cc("BGRA")) {
        const int c = (y * W + x) * 4;
        o[0] = im[c + 2] * s, o[1] = im[c + 1] * s, o[2] = im[c + 0] * s, o[3] = im[c + 3] * s;
        return VMO_OK;
    }
    if (format == cc("RGB3") || format == cc("RGB8")) {
        const int c = (y * W + x) * 3;
        o[0] = im[c + 0] * s, o[1] = im[c + 1] * s, o[2] = im[c + 2] * s, o[3] = real(1.0);
        return VMO_OK;
    }
    if (format == cc("RGBA")) {
        const int c = (y * W + x) * 4;
        o[0] = im[c + 0] * s, o[1] = im[c + 1] * s, o[2] = im[c + 2] * s, o[3] = im[c + 3] * s;
        return VMO_OK;
    }
    if (format == cc("GRAY") || format == cc("GREY") || format == cc("Y8  ")) {
        const int c = y * W + x;
        o[0] = o[1] = o[2] = im[c] * s, o[3] = real(1.0);
        return VMO_OK;
    }
    return VMO_ERR_FORMAT;
}

/* engine/cpu/pixel.hpp:115-144 */
int interpolate(const real* P, const uint8_t* im, int W, int H, uint32_t format, real* out) {
    const real x = P[0], y = P[1];
    const int x1 = std::max(int(std::floor(P[0])), 0);
    const int y1 = std::max(int(std::floor(P[1])), 0);
    const int x2 = std::min(x1 + 1, W - 1);
    const int y2 = std::min(y1 + 1, H - 1);
    real Q1[4], Q2[4], Q3[4], Q4[4];
    int rc;
    if ((rc = get_pixel(x1, y1, im, W, H, format, Q1)) != VMO_OK) return rc;
    if ((rc = get_pixel(x2, y1, im, W, H, format, Q2)) != VMO_OK) return rc;
    if ((rc = get_pixel(x1, y2, im, W, H, format, Q3)) != VMO_OK) return rc;
    if ((rc = get_pixel(x2, y2, im, W, H, format, Q4)) != VMO_OK) return rc;
    const real wx_a = (x2 - x) / (x2 - x1), wx_b = (x - x1) / (x2 - x1);
    const real wy_a = (y2 - y) / (y2 - y1), wy_b = (y - y1) / (y2 - y1);
    for (int c = 0; c < 4; ++c) {
        const real R1 = Q1[c] * wx_a + Q2[c] * wx_b;
        const real R2 = Q3[c] * wx_a + Q4[c] * wx_b;
        out[c] = R1 * wy_a + R2 * wy_b;
    }
    return VMO_OK;
}

/* engine/cpu/apply_activation.hpp:34-84 */
void apply_activation(int fn, real* d, size_t n_rows, int dims) {
    const size_t total = n_rows * size_t(dims);
    switch (fn) {
        case VMO_SELU: {
            const real lambda = 1.0507009873554804934193349852946;
            const real alpha = 1.6732632423543772848170429916717;
            for (size_t i = 0; i < total; ++i) d[i] = lambda * (d[i] >= 0 ? d[i] : alpha * std::exp(d[i]) - alpha);
        } break;
        case VMO_RELU:
            for (size_t i = 0; i < total; ++i) d[i] = std::max(d[i], real(0.0));
            break;
        case VMO_TANH:
            for (size_t i = 0; i < total; ++i) d[i] = std::tanh(d[i]);
            break;
        case VMO_SOFTMAX:
            for (size_t i = 0; i < total; ++i) d[i] = std::exp(d[i]);
            for (size_t r = 0; r < n_rows; ++r) {
                real* row = d + r * dims;
                real sum = real(0.0);
                for (int j = 0; j < dims; ++j) sum = sum + row[j];
                for (int j = 0; j < dims; ++j) row[j] = row[j] / sum;
            }
            break;
        default: break;
    }
}

/* engine/cpu/engine.hpp:84-147 */
int project_mesh(const vmo_mesh& mesh, const real* H, const vmo_lens& lens, int cap, real* px_out, int32_t* nb_out,
                 int32_t* gidx_out) {
    const std::vector<std::pair<int, int>> ranges = lookup(mesh, H, lens);
    const M3 Rco = rco_from_hoc(H);
    int cand = 0;
    for (const auto& r : ranges) cand += r.second - r.first;
    if (cand > cap) return VMO_ERR_CAPACITY;

    int V = 0;
    for (const auto& r : ranges) {
        for (int i = r.first; i < r.second; ++i) {
            const V2 px = project(mul(Rco, mesh.rays[i]), lens);
            if (0 <= px[0] && px[0] + 1 < lens.width && 0 <= px[1] && px[1] + 1 < lens.height) {
                gidx_out[V] = i;
                px_out[2 * V] = px[0];
                px_out[2 * V + 1] = px[1];
                ++V;
            }
        }
    }
    const int nn = mesh.nn;
    std::vector<int> r_lookup(size_t(mesh.n()) + 1, V);
    for (int i = 0; i < V; ++i) r_lookup[gidx_out[i]] = i;
    for (int i = 0; i < V; ++i)
        for (int j = 0; j < nn; ++j) nb_out[size_t(i) * nn + j] = r_lookup[mesh.nbr[size_t(gidx_out[i]) * nn + j]];
    for (int j = 0; j < nn; ++j) nb_out[size_t(V) * nn + j] = V;
    return V;
}

/* engine/cpu/engine.hpp:180-273, with input/output as locals so every call starts from empty buffers
 * (the reference keeps them as members and never clears input, which makes every call after the first on
 * one engine object wrong; a fresh reference engine per call is what this equals). */
int classify_mesh(const vmo_mesh& mesh, const real* H, const vmo_lens& lens, const void* image, uint32_t format,
                  const vmo_network* net, int cap, real* px, int32_t* nb, int32_t* gidx, real* cls) {
    const int V = project_mesh(mesh, H, lens, cap, px, nb, gidx);
    if (V <= 0) return V;
    const int nn = mesh.nn;
    const size_t n_points = size_t(V) + 1;
    const uint8_t* im = reinterpret_cast<const uint8_t*>(image);

    std::vector<real> input(n_points * 4), output;
    for (int i = 0; i < V; ++i) {
        const int rc = interpolate(px + 2 * size_t(i), im, lens.width, lens.height, format, &input[size_t(i) * 4]);
        if (rc != VMO_OK) return rc;
    }
    for (int c = 0; c < 4; ++c) input[size_t(V) * 4 + c] = -real(1.0);

    int in_dims = 4;
    int layer_index = 0;
    for (int g = 0; net != nullptr && g < net->n_groups; ++g) {
        /* gather: [self, neighbour 0 .. neighbour nn-1] */
        const int gathered = in_dims * (nn + 1);
        output.resize(n_points * gathered);
        for (size_t i = 0; i < n_points; ++i) {
            real* o = &output[i * gathered];
            std::memcpy(o, &input[i * in_dims], sizeof(real) * in_dims);
            for (int j = 0; j < nn; ++j)
                std::memcpy(o + (j + 1) * in_dims, &input[size_t(nb[i * nn + j]) * in_dims], sizeof(real) * in_dims);
        }
        std::swap(input, output);
        in_dims = gathered;

        for (int l = 0; l < net->group_sizes[g]; ++l, ++layer_index) {
            const vmo_layer& L = net->layers[layer_index];
            if (L.n_in != in_dims) return VMO_ERR_ARG;
            const int out_dims = L.n_out;
            /* transposed copy, engine/cpu/engine.hpp:57-71 */
            std::vector<real> wT(size_t(out_dims) * in_dims);
            for (int t = 0; t < in_dims; ++t)
                for (int j = 0; j < out_dims; ++j) wT[size_t(j) * in_dims + t] = L.weights[size_t(t) * out_dims + j];
            output.resize(n_points * out_dims);
            for (size_t i = 0; i < n_points; ++i) {
                const real* in = &input[i * in_dims];
                for (int j = 0; j < out_dims; ++j) {
                    const real* w = &wT[size_t(j) * in_dims];
                    real acc = L.biases[j]; /* std::inner_product: acc = acc + a*b, in order */
                    for (int t = 0; t < in_dims; ++t) acc = acc + in[t] * w[t];
                    output[i * out_dims + j] = acc;
                }
            }
            apply_activation(L.activation, output.data(), n_points, out_dims);
            std::swap(input, output);
            in_dims = out_dims;
        }
    }
    std::memcpy(cls, input.data(), sizeof(real) * n_points * in_dims);
    return V;
}

}  // namespace

/* ------------------------------------------------------------------ C interface */
struct vmo_visualmesh {
    std::map<real, vmo_mesh*> luts;
    std::vector<vmo_mesh*> ordered;
};

extern "C" {

const char* vmo_name(void) { return "oracle"; }

vmo_mesh* vmo_mesh_create(int model, int shape, real radius, real h, real k, real max_distance) {
    if ((model != VMO_MODEL_RING6 && model != VMO_MODEL_NMGRID8) || (shape != VMO_SHAPE_SPHERE && shape != VMO_SHAPE_CIRCLE))
        return nullptr;
    vmo_mesh* m = new vmo_mesh();
    try {
        const Shape s{shape, radius};
        m->h = h;
        m->max_distance = max_distance;
        if (model == VMO_MODEL_RING6) generate_ring6(*m, s, h, k, max_distance);
        else generate_nmgrid8(*m, s, h, k, max_distance);
        finish_mesh(*m);
    } catch (...) {
        delete m;
        return nullptr;
    }
    return m;
}
void vmo_mesh_destroy(vmo_mesh* m) { delete m; }
int vmo_mesh_n_nodes(const vmo_mesh* m) { return m->n(); }
int vmo_mesh_n_neighbours(const vmo_mesh* m) { return m->nn; }
real vmo_mesh_h(const vmo_mesh* m) { return m->h; }
void vmo_mesh_copy(const vmo_mesh* m, real* rays, int32_t* neighbours) {
    if (rays) std::memcpy(rays, m->rays.data(), sizeof(real) * 3 * m->rays.size());
    if (neighbours) std::memcpy(neighbours, m->nbr.data(), sizeof(int32_t) * m->nbr.size());
}
int vmo_mesh_lookup(const vmo_mesh* m, const real* Hoc16, const vmo_lens* lens, int32_t* ranges, int cap) {
    try {
        const std::vector<std::pair<int, int>> r = lookup(*m, Hoc16, *lens);
        for (int i = 0; i < int(r.size()) && i < cap; ++i) {
            ranges[2 * i] = r[i].first;
            ranges[2 * i + 1] = r[i].second;
        }
        return int(r.size());
    } catch (...) { return VMO_ERR_LENS; }
}

/* visualmesh.hpp:64-96 */
vmo_visualmesh* vmo_visualmesh_create(int model, int shape, real radius, real min_h, real max_h, real k,
                                      real max_error, real max_distance) {
    vmo_visualmesh* v = new vmo_visualmesh();
    const Shape s{shape, radius};
    auto add = [&](real h) {
        if (v->luts.count(h)) return true; /* std::map::insert keeps the first */
        vmo_mesh* m = vmo_mesh_create(model, shape, radius, h, k, max_distance);
        if (!m) return false;
        v->luts[h] = m;
        return true;
    };
    bool ok = add(min_h) && add(max_h);
    std::vector<V2> stack;
    stack.push_back(V2{{min_h, max_h}});
    while (ok && !stack.empty()) {
        const V2 range = stack.back();
        const real h = (range[0] + range[1]) / 2;
        stack.pop_back();
        const real lower_err = std::abs(k - k * s.k(range[0], h));
        const real upper_err = std::abs(k - k * s.k(range[1], h));
        if (lower_err > max_error || upper_err > max_error) {
            ok = add(h);
            stack.push_back(V2{{range[0], h}});
            stack.push_back(V2{{h, range[1]}});
        }
    }
    if (!ok) {
        vmo_visualmesh_destroy(v);
        return nullptr;
    }
    for (auto& kv : v->luts) v->ordered.push_back(kv.second);
    return v;
}
void vmo_visualmesh_destroy(vmo_visualmesh* v) {
    if (!v) return;
    for (auto& kv : v->luts) delete kv.second;
    delete v;
}
int vmo_visualmesh_n_meshes(const vmo_visualmesh* v) { return int(v->ordered.size()); }
const vmo_mesh* vmo_visualmesh_mesh(const vmo_visualmesh* v, int i) { return v->ordered[i]; }
/* visualmesh.hpp:122-135 */
const vmo_mesh* vmo_visualmesh_height(const vmo_visualmesh* v, real h) {
    auto it = v->luts.lower_bound(h);
    if (it == v->luts.begin()) return it->second;
    if (it == v->luts.end()) return v->luts.rbegin()->second;
    auto pv = std::prev(it);
    return std::abs(it->first - h) < std::abs(pv->first - h) ? it->second : pv->second;
}

int vmo_project(const vmo_mesh* m, const real* Hoc16, const vmo_lens* lens, int cap, real* px, int32_t* nb,
                int32_t* gidx) {
    try {
        return project_mesh(*m, Hoc16, *lens, cap, px, nb, gidx);
    } catch (...) { return VMO_ERR_LENS; }
}
int vmo_classify(const vmo_mesh* m, const real* Hoc16, const vmo_lens* lens, const void* image, uint32_t fourcc,
                 const vmo_network* net, int cap, real* px, int32_t* nb, int32_t* gidx, real* cls) {
    try {
        return classify_mesh(*m, Hoc16, *lens, image, fourcc, net, cap, px, nb, gidx, cls);
    } catch (...) { return VMO_ERR_LENS; }
}

void vmo_fn_project(const real* r, const vmo_lens* lens, real* px2) {
    const V2 p = project(V3{{r[0], r[1], r[2]}}, *lens);
    px2[0] = p[0], px2[1] = p[1];
}
void vmo_fn_unproject(const real* px2, const vmo_lens* lens, real* ray3) {
    const V3 r = unproject(V2{{px2[0], px2[1]}}, *lens);
    ray3[0] = r[0], ray3[1] = r[1], ray3[2] = r[2];
}
int vmo_fn_interpolate(const real* px2, const void* image, int width, int height, uint32_t fourcc, real* out4) {
    return interpolate(px2, reinterpret_cast<const uint8_t*>(image), width, height, fourcc, out4);
}
int vmo_fn_get_pixel(int x, int y, const void* image, int width, int height, uint32_t fourcc, real* out4) {
    return get_pixel(x, y, reinterpret_cast<const uint8_t*>(image), width, height, fourcc, out4);
}
void vmo_fn_activation(int activation, real* data, int n_rows, int dims) {
    apply_activation(activation, data, size_t(n_rows), dims);
}
real vmo_fn_shape(int shape, real radius, int which, real a, real b) {
    const Shape s{shape, radius};
    switch (which) {
        case 0: return s.phi(a, b);
        case 1: return s.n(a, b);
        case 2: return s.theta(a, b);
        case 3: return s.k(a, b);
        default: return s.c();
    }
}
void vmo_fn_libm(int which, const real* x, real* y, int n) {
    for (int i = 0; i < n; ++i)
        y[i] = which == 0 ? std::acos(x[i]) : which == 1 ? std::sin(x[i]) : which == 2 ? std::tan(x[i]) : std::sqrt(x[i]);
}
}

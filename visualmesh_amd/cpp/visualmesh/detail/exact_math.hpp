/*
 * fp32 vector helpers with a fixed operation order.
 *
 * The node order of a mesh, the lookup ranges and the visible set all depend on last-bit comparisons of
 * fp32 results, so the host code must evaluate every expression in the reference's order
 * (reference utility/math.hpp: dot is a[n-1]*b[n-1] + dot of the leading components, :145-164; norm,
 * normalise, cross :166-184; 3x3 inverse :275-301). Compile host code that includes this header with
 * -ffp-contract=off and without -ffast-math.
 */
#ifndef VISUALMESH_DETAIL_EXACT_MATH_HPP
#define VISUALMESH_DETAIL_EXACT_MATH_HPP

#include <cmath>
#include <limits>

#include "../types.hpp"

namespace visualmesh {
namespace detail {

    typedef vec2<float> f2;
    typedef vec3<float> f3;

    inline float dot(const f2& a, const f2& b) { return a[1] * b[1] + a[0] * b[0]; }
    inline float dot(const f3& a, const f3& b) { return a[2] * b[2] + (a[1] * b[1] + a[0] * b[0]); }
    inline float length(const f3& a) { return std::sqrt(dot(a, a)); }
    inline f3 unit(const f3& a) {
        const float inv = 1.0f / length(a);
        return f3{{a[0] * inv, a[1] * inv, a[2] * inv}};
    }
    inline f3 cross(const f3& a, const f3& b) {
        return f3{{a[1] * b[2] - a[2] * b[1], a[2] * b[0] - a[0] * b[2], a[0] * b[1] - a[1] * b[0]}};
    }
    inline f3 apply(const mat3<float>& m, const f3& v) { return f3{{dot(m[0], v), dot(m[1], v), dot(m[2], v)}}; }

    /// Rotation observation-plane -> camera: the transpose of Hoc's rotation block.
    inline mat3<float> rotation_co(const mat4<float>& Hoc) {
        mat3<float> r;
        for (int i = 0; i < 3; ++i)
            for (int j = 0; j < 3; ++j) r[i][j] = Hoc[j][i];
        return r;
    }
    /// Rotation camera -> observation-plane: Hoc's rotation block.
    inline mat3<float> rotation_oc(const mat4<float>& Hoc) {
        mat3<float> r;
        for (int i = 0; i < 3; ++i)
            for (int j = 0; j < 3; ++j) r[i][j] = Hoc[i][j];
        return r;
    }

    /// A cone around `axis` with half angle acos(c); s = sin of the half angle where it is kept.
    struct Cone {
        f3 axis;
        float c;
        float s;
    };

    /// Cones through one, two and three unit vectors (reference utility/cone.hpp:32-98).
    inline Cone cone_through() { return Cone{f3{{0, 0, 0}}, 1, 0}; }
    inline Cone cone_through(const f3& p) { return Cone{p, 1, 0}; }
    inline Cone cone_through(const f3& p, const f3& q) {
        const f3 axis = unit(f3{{p[0] + q[0], p[1] + q[1], p[2] + q[2]}});
        return Cone{axis, dot(axis, p), 0};
    }
    inline Cone cone_through(const f3& p, const f3& q, const f3& r) {
        const f3 m[3] = {p, q, r};
        const float det = (m[0][0] * (m[1][1] * m[2][2] - m[2][1] * m[1][2]) - m[0][1] * (m[1][0] * m[2][2] - m[1][2] * m[2][0])
                           + m[0][2] * (m[1][0] * m[2][1] - m[1][1] * m[2][0]));
        f3 inv[3];
        if (det == 0) {
            const float nan = std::numeric_limits<float>::quiet_NaN();
            inv[0] = inv[1] = inv[2] = f3{{nan, nan, nan}};
        }
        else {
            const float idet = 1.0f / det;
            inv[0] = f3{{(m[1][1] * m[2][2] - m[2][1] * m[1][2]) * idet, (m[0][2] * m[2][1] - m[0][1] * m[2][2]) * idet,
                         (m[0][1] * m[1][2] - m[0][2] * m[1][1]) * idet}};
            inv[1] = f3{{(m[1][2] * m[2][0] - m[1][0] * m[2][2]) * idet, (m[0][0] * m[2][2] - m[0][2] * m[2][0]) * idet,
                         (m[1][0] * m[0][2] - m[0][0] * m[1][2]) * idet}};
            inv[2] = f3{{(m[1][0] * m[2][1] - m[2][0] * m[1][1]) * idet, (m[2][0] * m[0][1] - m[0][0] * m[2][1]) * idet,
                         (m[0][0] * m[1][1] - m[1][0] * m[0][1]) * idet}};
        }
        const f3 one{{1, 1, 1}};
        const f3 axis = unit(f3{{dot(inv[0], one), dot(inv[1], one), dot(inv[2], one)}});
        return Cone{axis, dot(axis, p), 0};
    }
    inline Cone with_sine(Cone k) {
        k.s = std::sqrt(1.0f - k.c * k.c);
        return k;
    }

}  // namespace detail
}  // namespace visualmesh

#endif  // VISUALMESH_DETAIL_EXACT_MATH_HPP

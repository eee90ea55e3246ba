/*
 * Vector helpers with a fixed operation order, for T = float or double (the reference's Scalar).
 *
 * The node order of a mesh, the lookup ranges and the visible set all depend on last-bit comparisons of
 * results in T, so the host code must evaluate every expression in the reference's order
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


    template <typename T>
    inline T dot(const vec2<T>& a, const vec2<T>& b) { return a[1] * b[1] + a[0] * b[0]; }
    template <typename T>
    inline T dot(const vec3<T>& a, const vec3<T>& b) { return a[2] * b[2] + (a[1] * b[1] + a[0] * b[0]); }
    template <typename T>
    inline T length(const vec3<T>& a) { return std::sqrt(dot(a, a)); }
    template <typename T>
    inline vec3<T> unit(const vec3<T>& a) {
        const T inv = T(1.0) / length(a);
        return vec3<T>{{a[0] * inv, a[1] * inv, a[2] * inv}};
    }
    template <typename T>
    inline vec3<T> cross(const vec3<T>& a, const vec3<T>& b) {
        return vec3<T>{{a[1] * b[2] - a[2] * b[1], a[2] * b[0] - a[0] * b[2], a[0] * b[1] - a[1] * b[0]}};
    }
    template <typename T>
    inline vec3<T> apply(const mat3<T>& m, const vec3<T>& v) { return vec3<T>{{dot(m[0], v), dot(m[1], v), dot(m[2], v)}}; }

    /// Rotation observation-plane -> camera: the transpose of Hoc's rotation block.
    template <typename T>
    inline mat3<T> rotation_co(const mat4<T>& Hoc) {
        mat3<T> r;
        for (int i = 0; i < 3; ++i)
            for (int j = 0; j < 3; ++j) r[i][j] = Hoc[j][i];
        return r;
    }
    /// Rotation camera -> observation-plane: Hoc's rotation block.
    template <typename T>
    inline mat3<T> rotation_oc(const mat4<T>& Hoc) {
        mat3<T> r;
        for (int i = 0; i < 3; ++i)
            for (int j = 0; j < 3; ++j) r[i][j] = Hoc[i][j];
        return r;
    }

    /// A cone around `axis` with half angle acos(c); s = sin of the half angle where it is kept.
    template <typename T>
    struct ConeT {
        vec3<T> axis;
        T c;
        T s;
    };

    /// Cones through one, two and three unit vectors (reference utility/cone.hpp:32-98).
    template <typename T>
    inline ConeT<T> cone_through() { return ConeT<T>{vec3<T>{{0, 0, 0}}, 1, 0}; }
    template <typename T>
    inline ConeT<T> cone_through(const vec3<T>& p) { return ConeT<T>{p, 1, 0}; }
    template <typename T>
    inline ConeT<T> cone_through(const vec3<T>& p, const vec3<T>& q) {
        const vec3<T> axis = unit(vec3<T>{{p[0] + q[0], p[1] + q[1], p[2] + q[2]}});
        return ConeT<T>{axis, dot(axis, p), 0};
    }
    template <typename T>
    inline ConeT<T> cone_through(const vec3<T>& p, const vec3<T>& q, const vec3<T>& r) {
        const vec3<T> m[3] = {p, q, r};
        const T det = (m[0][0] * (m[1][1] * m[2][2] - m[2][1] * m[1][2]) - m[0][1] * (m[1][0] * m[2][2] - m[1][2] * m[2][0])
                           + m[0][2] * (m[1][0] * m[2][1] - m[1][1] * m[2][0]));
        vec3<T> inv[3];
        if (det == 0) {
            const T nan = std::numeric_limits<T>::quiet_NaN();
            inv[0] = inv[1] = inv[2] = vec3<T>{{nan, nan, nan}};
        }
        else {
            const T idet = T(1.0) / det;
            inv[0] = vec3<T>{{(m[1][1] * m[2][2] - m[2][1] * m[1][2]) * idet, (m[0][2] * m[2][1] - m[0][1] * m[2][2]) * idet,
                         (m[0][1] * m[1][2] - m[0][2] * m[1][1]) * idet}};
            inv[1] = vec3<T>{{(m[1][2] * m[2][0] - m[1][0] * m[2][2]) * idet, (m[0][0] * m[2][2] - m[0][2] * m[2][0]) * idet,
                         (m[1][0] * m[0][2] - m[0][0] * m[1][2]) * idet}};
            inv[2] = vec3<T>{{(m[1][0] * m[2][1] - m[2][0] * m[1][1]) * idet, (m[2][0] * m[0][1] - m[0][0] * m[2][1]) * idet,
                         (m[0][0] * m[1][1] - m[1][0] * m[0][1]) * idet}};
        }
        const vec3<T> one{{1, 1, 1}};
        const vec3<T> axis = unit(vec3<T>{{dot(inv[0], one), dot(inv[1], one), dot(inv[2], one)}});
        return ConeT<T>{axis, dot(axis, p), 0};
    }
    template <typename T>
    inline ConeT<T> with_sine(ConeT<T> k) {
        k.s = std::sqrt(T(1.0) - k.c * k.c);
        return k;
    }

    typedef vec2<float> f2;
    typedef vec3<float> f3;
    typedef ConeT<float> Cone;

}  // namespace detail
}  // namespace visualmesh

#endif  // VISUALMESH_DETAIL_EXACT_MATH_HPP

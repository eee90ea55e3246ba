/*
 * Lens projection and its inverse on the host, in the reference's arithmetic for Scalar = T (float or double)
 * (reference utility/projection.hpp: lens radius functions :26-60, distortion :79-144,
 * project :162-187, unproject :204-225). The device kernels evaluate the same expressions; the host
 * versions serve the BSP lookup and the re-decision of nodes that project onto a screen edge.
 */
#ifndef VISUALMESH_DETAIL_LENS_MATH_HPP
#define VISUALMESH_DETAIL_LENS_MATH_HPP

#include <algorithm>
#include <cmath>
#include <stdexcept>

#include "exact_math.hpp"

namespace visualmesh {
namespace detail {

    /// r_d = r * (1 + ik0 r^2 + ik1 r^4 + ik2 r^6 + ik3 r^8): T terms summed in double (the reference's literal 1.0), rounded once to T.
    template <typename T>
    inline T radial_distort(T r, const std::array<T, 2>& k) {
        const T i0 = -k[0];
        const T i1 = T(3.0) * (k[0] * k[0]) - k[1];
        const T i2 = -T(12.0) * (k[0] * k[0]) * k[0] + T(8.0) * k[0] * k[1];
        const T i3 = T(55.0) * (k[0] * k[0]) * (k[0] * k[0]) - T(55.0) * (k[0] * k[0]) * k[1] + T(5.0) * (k[1] * k[1]);
        const T r2 = r * r;
        const double bracket = 1.0 + double(i0 * r2) + double(i1 * (r2 * r2)) + double(i2 * (r2 * r2) * r2)
                               + double(i3 * (r2 * r2) * (r2 * r2));
        return T(double(r) * bracket);
    }
    template <typename T>
    inline T radial_undistort(T r, const std::array<T, 2>& k) {
        const T r2 = r * r;
        return T(double(r) * (1.0 + double(k[0] * r2) + double(k[1] * (r2 * r2))));
    }

    /// Camera-space unit vector (x forward, y left, z up) -> pixel (origin top left, x right, y down).
    template <typename T>
    inline vec2<T> project(const vec3<T>& ray, const Lens<T>& lens) {
        const T f = lens.focal_length;
        const T theta = std::acos(ray[0]);
        const T inv_sin = T(1.0) / std::sqrt(T(1.0) - ray[0] * ray[0]);
        T r_u;
        switch (lens.projection) {
            case RECTILINEAR: r_u = f * std::tan(std::min(std::max(theta, T(0.0)), T(M_PI_2))); break;
            case EQUISOLID: r_u = T(2.0) * f * std::sin(theta * T(0.5)); break;
            case EQUIDISTANT: r_u = f * theta; break;
            default: throw std::runtime_error("Cannot project: Unknown lens type");
        }
        const T r_d = radial_distort(r_u, lens.k);
        vec2<T> screen{{T(0.0), T(0.0)}};
        if (!(ray[0] >= 1)) screen = vec2<T>{{r_d * ray[1] * inv_sin, r_d * ray[2] * inv_sin}};
        return vec2<T>{{(T(lens.dimensions[0]) * T(0.5) - screen[0]) - lens.centre[0],
                   (T(lens.dimensions[1]) * T(0.5) - screen[1]) - lens.centre[1]}};
    }

    /// Pixel -> camera-space unit vector.
    template <typename T>
    inline vec3<T> unproject(const vec2<T>& px, const Lens<T>& lens) {
        const vec2<T> screen{{T(lens.dimensions[0]) * T(0.5) - (px[0] + lens.centre[0]),
                         T(lens.dimensions[1]) * T(0.5) - (px[1] + lens.centre[1])}};
        const T f = lens.focal_length;
        const T r_d = std::sqrt(dot(screen, screen));
        if (r_d == 0) return vec3<T>{{T(1.0), T(0.0), T(0.0)}};
        const T r_u = radial_undistort(r_d, lens.k);
        T theta;
        switch (lens.projection) {
            case RECTILINEAR: theta = std::atan(r_u / f); break;
            case EQUISOLID: theta = T(2.0) * std::asin(r_u / (T(2.0) * f)); break;
            case EQUIDISTANT: theta = r_u / f; break;
            default: throw std::runtime_error("Cannot project: Unknown lens type");
        }
        const T st = std::sin(theta);
        return vec3<T>{{std::cos(theta), st * screen[0] / r_d, st * screen[1] / r_d}};
    }

}  // namespace detail
}  // namespace visualmesh

#endif  // VISUALMESH_DETAIL_LENS_MATH_HPP

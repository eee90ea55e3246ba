/*
 * Lens projection and its inverse on the host, in the reference's fp32 arithmetic
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

    /// r_d = r * (1 + ik0 r^2 + ik1 r^4 + ik2 r^6 + ik3 r^8): float terms summed in double, rounded once.
    inline float radial_distort(float r, const std::array<float, 2>& k) {
        const float i0 = -k[0];
        const float i1 = 3.0f * (k[0] * k[0]) - k[1];
        const float i2 = -12.0f * (k[0] * k[0]) * k[0] + 8.0f * k[0] * k[1];
        const float i3 = 55.0f * (k[0] * k[0]) * (k[0] * k[0]) - 55.0f * (k[0] * k[0]) * k[1] + 5.0f * (k[1] * k[1]);
        const float r2 = r * r;
        const double bracket = 1.0 + double(i0 * r2) + double(i1 * (r2 * r2)) + double(i2 * (r2 * r2) * r2)
                               + double(i3 * (r2 * r2) * (r2 * r2));
        return float(double(r) * bracket);
    }
    inline float radial_undistort(float r, const std::array<float, 2>& k) {
        const float r2 = r * r;
        return float(double(r) * (1.0 + double(k[0] * r2) + double(k[1] * (r2 * r2))));
    }

    /// Camera-space unit vector (x forward, y left, z up) -> pixel (origin top left, x right, y down).
    inline f2 project(const f3& ray, const Lens<float>& lens) {
        const float f = lens.focal_length;
        const float theta = std::acos(ray[0]);
        const float inv_sin = 1.0f / std::sqrt(1.0f - ray[0] * ray[0]);
        float r_u;
        switch (lens.projection) {
            case RECTILINEAR: r_u = f * std::tan(std::min(std::max(theta, 0.0f), float(M_PI_2))); break;
            case EQUISOLID: r_u = 2.0f * f * std::sin(theta * 0.5f); break;
            case EQUIDISTANT: r_u = f * theta; break;
            default: throw std::runtime_error("Cannot project: Unknown lens type");
        }
        const float r_d = radial_distort(r_u, lens.k);
        f2 screen{{0.0f, 0.0f}};
        if (!(ray[0] >= 1)) screen = f2{{r_d * ray[1] * inv_sin, r_d * ray[2] * inv_sin}};
        return f2{{(float(lens.dimensions[0]) * 0.5f - screen[0]) - lens.centre[0],
                   (float(lens.dimensions[1]) * 0.5f - screen[1]) - lens.centre[1]}};
    }

    /// Pixel -> camera-space unit vector.
    inline f3 unproject(const f2& px, const Lens<float>& lens) {
        const f2 screen{{float(lens.dimensions[0]) * 0.5f - (px[0] + lens.centre[0]),
                         float(lens.dimensions[1]) * 0.5f - (px[1] + lens.centre[1])}};
        const float f = lens.focal_length;
        const float r_d = std::sqrt(dot(screen, screen));
        if (r_d == 0) return f3{{1.0f, 0.0f, 0.0f}};
        const float r_u = radial_undistort(r_d, lens.k);
        float theta;
        switch (lens.projection) {
            case RECTILINEAR: theta = std::atan(r_u / f); break;
            case EQUISOLID: theta = 2.0f * std::asin(r_u / (2.0f * f)); break;
            case EQUIDISTANT: theta = r_u / f; break;
            default: throw std::runtime_error("Cannot project: Unknown lens type");
        }
        const float st = std::sin(theta);
        return f3{{std::cos(theta), st * screen[0] / r_d, st * screen[1] / r_d}};
    }

}  // namespace detail
}  // namespace visualmesh

#endif  // VISUALMESH_DETAIL_LENS_MATH_HPP

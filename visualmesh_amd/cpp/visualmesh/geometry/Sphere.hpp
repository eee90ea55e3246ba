/*
 * Sphere of radius r resting on the observation plane: the shape functions a mesh generator needs
 * (reference geometry/Sphere.hpp:55-134). Operand types follow the reference for Scalar = float and double alike so that the
 * generated mesh is bit-identical.
 */
#ifndef VISUALMESH_GEOMETRY_SPHERE_HPP
#define VISUALMESH_GEOMETRY_SPHERE_HPP

#include <cmath>
#include <type_traits>

namespace visualmesh {
namespace geometry {

    template <typename Scalar>
    struct Sphere {
        explicit Sphere(const Scalar& radius) : r(radius) {}

        /// angle from straight down to the centre of the n-th object
        Scalar phi(const Scalar& n, const Scalar& h) const { return -std::atan(std::sinh(n * std::log1p(-Scalar(2.0) * r / h))); }
        /// inverse of phi
        Scalar n(const Scalar& phi_, const Scalar& h) const { return std::asinh(std::tan(-phi_)) / std::log1p(-Scalar(2.0) * r / h); }
        /// ratio of intersections seen from h1 versus h0
        Scalar k(const Scalar& h0, const Scalar& h1) const {
            return (std::log(h1 - 2 * r) - std::log(h1)) / (std::log(h0 - 2 * r) - std::log(h0));
        }
        /// height of the object's centre above the plane
        const Scalar& c() const { return r; }
        /// angular width of the object at ring n. Below n = 0.5 it is interpolated from 2 pi to pi; that arm
        /// divides in double and both arms meet in double before the result is rounded.
        Scalar theta(const Scalar& n, const Scalar& h) const {
            const double v = n <= 0.5 ? double(Scalar(2.0 * M_PI)) / (1.0 + double(n * Scalar(2.0)))
                                      : double(Scalar(2.0) * std::asin(r / ((h - r) * std::tan(phi(n, h)))));
            return Scalar(v);
        }

        Scalar r;
    };

}  // namespace geometry
}  // namespace visualmesh

#endif  // VISUALMESH_GEOMETRY_SPHERE_HPP

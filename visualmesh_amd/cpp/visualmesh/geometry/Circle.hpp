/*
 * Flat circle of radius r lying on the observation plane (reference geometry/Circle.hpp:62-138).
 * Operand types follow the reference for Scalar = float and double alike so that the generated mesh is bit-identical.
 */
#ifndef VISUALMESH_GEOMETRY_CIRCLE_HPP
#define VISUALMESH_GEOMETRY_CIRCLE_HPP

#include <cmath>
#include <type_traits>

namespace visualmesh {
namespace geometry {

    template <typename Scalar>
    struct Circle {
        explicit Circle(const Scalar& radius) : r(radius) {}

        Scalar phi(const Scalar& n, const Scalar& h) const { return std::atan((Scalar(2.0) * n * r) / h); }
        Scalar n(const Scalar& phi_, const Scalar& h) const { return (h * std::tan(phi_)) / (Scalar(2.0) * r); }
        Scalar k(const Scalar& h0, const Scalar& h1) const { return h0 / h1; }
        Scalar c() const { return Scalar(0.0); }
        Scalar theta(const Scalar& n, const Scalar& h) const {
            const double v = n <= 0.5 ? double(Scalar(2.0 * M_PI)) / (1.0 + double(n * Scalar(2.0)))
                                      : double(Scalar(2.0) * std::asin(r / ((h - r) * std::tan(phi(n, h)))));
            return Scalar(v);
        }

        Scalar r;
    };

}  // namespace geometry
}  // namespace visualmesh

#endif  // VISUALMESH_GEOMETRY_CIRCLE_HPP

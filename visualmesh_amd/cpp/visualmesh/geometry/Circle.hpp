/*
 * Flat circle of radius r lying on the observation plane (reference geometry/Circle.hpp:62-138).
 * fp32 only; operand types follow the reference so that the generated mesh is bit-identical.
 */
#ifndef VISUALMESH_GEOMETRY_CIRCLE_HPP
#define VISUALMESH_GEOMETRY_CIRCLE_HPP

#include <cmath>
#include <type_traits>

namespace visualmesh {
namespace geometry {

    template <typename Scalar>
    struct Circle {
        static_assert(std::is_same<Scalar, float>::value, "the host mesh code is written for float");
        explicit Circle(const Scalar& radius) : r(radius) {}

        Scalar phi(const Scalar& n, const Scalar& h) const { return std::atan((2.0f * n * r) / h); }
        Scalar n(const Scalar& phi_, const Scalar& h) const { return (h * std::tan(phi_)) / (2.0f * r); }
        Scalar k(const Scalar& h0, const Scalar& h1) const { return h0 / h1; }
        Scalar c() const { return 0.0f; }
        Scalar theta(const Scalar& n, const Scalar& h) const {
            const double v = n <= 0.5 ? double(float(2.0 * M_PI)) / (1.0 + double(n * 2.0f))
                                      : double(2.0f * std::asin(r / ((h - r) * std::tan(phi(n, h)))));
            return float(v);
        }

        Scalar r;
    };

}  // namespace geometry
}  // namespace visualmesh

#endif  // VISUALMESH_GEOMETRY_CIRCLE_HPP

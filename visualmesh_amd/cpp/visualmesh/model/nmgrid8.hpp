/*
 * NMGrid8 mesh generator: a square grid in "object count" coordinates (n objects along x, m along y) with
 * eight neighbours per node, grown by flood fill from the point below the camera.
 * Follows reference model/grid_base.hpp:78-144 (flood fill order and neighbour table, with the 8-neighbour
 * offsets :65-74) and model/nmgrid_map.hpp:33-131 (coordinates -> vector by bisection on the plane height)
 * operation for operation in Scalar (float or double). The visit order of the fill (a LIFO stack and the offset order) fixes
 * the node numbering; the containers used for membership do not.
 */
#ifndef VISUALMESH_MODEL_NMGRID8_HPP
#define VISUALMESH_MODEL_NMGRID8_HPP

#include <array>
#include <cmath>
#include <cstdint>
#include <type_traits>
#include <unordered_map>
#include <vector>

#include "../types.hpp"

namespace visualmesh {
namespace model {

    template <typename Scalar>
    struct NMGrid8 {
        static constexpr int N_NEIGHBOURS = 8;
        typedef Node<Scalar, N_NEIGHBOURS> node_type;

    private:
        /// Ground point seen n objects out along x on the plane whose own camera height would be h_n.
        template <typename Shape>
        static vec3<Scalar> ground_point(const Shape& shape, const Scalar h, const Scalar n, const Scalar h_n) {
            const Scalar c = shape.c();
            const Scalar x = (h_n - c) * std::tan(shape.phi(n, h_n));
            const Scalar y = std::sqrt((h_n - c) * (h_n - c) - (h - c) * (h - c));
            return vec3<Scalar>{{x, y, c - h}};
        }
        /// The m coordinate that ground_point(n, h_n) corresponds to.
        template <typename Shape>
        static Scalar implied_m(const Shape& shape, const Scalar h, const Scalar n, const Scalar h_n) {
            const Scalar c = shape.c();
            const vec3<Scalar> v = ground_point(shape, h, n, h_n);
            const Scalar h_m = std::sqrt(v[0] * v[0] + v[2] * v[2]) + c;
            const Scalar phi_m = std::acos(std::sqrt((v[0] * v[0] + v[2] * v[2]) / (v[0] * v[0] + v[1] * v[1] + v[2] * v[2])));
            return shape.n(phi_m, h_m);
        }

    public:
        /// (n, m) -> vector to the object's centre (not normalised; z = c - h).
        template <typename Shape>
        static vec3<Scalar> map(const Shape& shape, const Scalar& h, const vec2<Scalar>& nm) {
            const Scalar n = std::abs(nm[0]);
            const Scalar m = std::abs(nm[1]);
            const Scalar c = shape.c();
            // bisect the plane height between "m = 0" and "n = 0"
            Scalar lo = h;
            Scalar hi = (h - c) / std::cos(shape.phi(m, h)) + c;
            Scalar h_n = Scalar(double(lo + hi) * 0.5);
            for (;;) {
                if (h_n == lo || h_n == hi) break;
                const Scalar guess = implied_m(shape, h, n, h_n);
                (guess > m ? hi : lo) = h_n;
                if (double(h_n) == double(lo + hi) * 0.5) break;
                h_n = Scalar(double(lo + hi) * 0.5);
            }
            vec3<Scalar> v = ground_point(shape, h, n, h_n);
            v[0] *= nm[0] >= 0 ? 1 : -1;
            v[1] *= nm[1] >= 0 ? 1 : -1;
            return v;
        }

        template <typename Shape>
        static std::vector<node_type> generate(const Shape& shape, const Scalar& h, const Scalar& k, const Scalar& max_distance) {
            static const int step[N_NEIGHBOURS][2] = {{-1, 0}, {-1, 1}, {0, 1}, {1, 1}, {1, 0}, {1, -1}, {0, -1}, {-1, -1}};
            const Scalar jump = Scalar(1.0 / double(k));
            auto key = [](int a, int b) { return (uint64_t(uint32_t(a)) << 32) | uint32_t(b); };

            std::vector<node_type> nodes;
            std::vector<std::array<int, 2>> coords;            // grid coordinate of each accepted node
            std::unordered_map<uint64_t, int> state;           // seen cells: -1 rejected/pending, else node index
            std::vector<std::array<int, 2>> pending(1, std::array<int, 2>{{0, 0}});
            state.emplace(key(0, 0), -1);
            while (!pending.empty()) {
                const std::array<int, 2> cell = pending.back();
                pending.pop_back();
                const vec3<Scalar> v = map(shape, h, vec2<Scalar>{{Scalar(cell[0]) * jump, Scalar(cell[1]) * jump}});
                const Scalar ground_distance = std::sqrt(v[1] * v[1] + v[0] * v[0]);
                if (ground_distance <= max_distance) {
                    node_type node{};
                    const Scalar inv = Scalar(1.0) / std::sqrt(v[2] * v[2] + (v[1] * v[1] + v[0] * v[0]));
                    node.ray = vec3<Scalar>{{v[0] * inv, v[1] * inv, v[2] * inv}};
                    state[key(cell[0], cell[1])] = int(nodes.size());
                    nodes.push_back(node);
                    coords.push_back(cell);
                    for (int t = 0; t < N_NEIGHBOURS; ++t) {
                        const std::array<int, 2> next{{cell[0] + step[t][0], cell[1] + step[t][1]}};
                        if (state.emplace(key(next[0], next[1]), -1).second) pending.push_back(next);
                    }
                }
            }
            const int total = int(nodes.size());
            for (int i = 0; i < total; ++i) {
                for (int t = 0; t < N_NEIGHBOURS; ++t) {
                    const auto it = state.find(key(coords[i][0] + step[t][0], coords[i][1] + step[t][1]));
                    nodes[i].neighbours[t] = (it != state.end() && it->second >= 0) ? it->second : total;
                }
            }
            return nodes;
        }
    };

}  // namespace model
}  // namespace visualmesh

#endif  // VISUALMESH_MODEL_NMGRID8_HPP

/*
 * Ring6 mesh generator: concentric rings of nodes around the point below the camera, six neighbours per
 * node (left, two on the next ring, right, two on the previous ring).
 * Follows reference model/ring_base.hpp:53-115 (ring spacing and sizes), model/ring6.hpp:50-69 (neighbour
 * offsets) and model/polar_map.hpp:41-72 (ring coordinates -> unit vector) operation for operation in Scalar (float or double):
 * ring sizes come from ceil() of quotients in Scalar, so any reordering changes the node count.
 */
#ifndef VISUALMESH_MODEL_RING6_HPP
#define VISUALMESH_MODEL_RING6_HPP

#include <algorithm>
#include <array>
#include <cmath>
#include <type_traits>
#include <vector>

#include "../types.hpp"

namespace visualmesh {
namespace model {

    template <typename Scalar>
    struct Ring6 {
        static constexpr int N_NEIGHBOURS = 6;
        typedef Node<Scalar, N_NEIGHBOURS> node_type;

        /// Offsets, relative to the first node of the current ring, of the six neighbours of the i-th
        /// node of a ring with `cur` nodes between rings of `prev` and `next` nodes.
        static std::array<int, N_NEIGHBOURS> neighbours(const int& i, const int& prev, const int& cur, const int& next) {
            const Scalar along = Scalar(i) / Scalar(cur);
            const int left = i > 0 ? i - 1 : cur - 1;
            const int right = i + 1 < cur ? i + 1 : 0;
            const int up = int(along * next);
            const int down = int(along * prev);
            return std::array<int, N_NEIGHBOURS>{{left, (up % next) + cur, ((up + 1) % next) + cur, right,
                                                  ((down + 1) % prev) - prev, (down % prev) - prev}};
        }

        /// Ring coordinates (n rings out, m objects around) -> unit vector.
        template <typename Shape>
        static vec3<Scalar> map(const Shape& shape, const Scalar& h, const vec2<Scalar>& nm) {
            const Scalar phi = shape.phi(std::abs(nm[0]), h);
            const Scalar step = shape.theta(std::abs(nm[0]), h);
            const Scalar theta = Scalar(double(step * nm[1]) + (nm[0] < 0 ? M_PI : 0.0));
            return vec3<Scalar>{{std::cos(theta) * std::sin(phi), std::sin(theta) * std::sin(phi), -std::cos(phi)}};
        }

        template <typename Shape>
        static std::vector<node_type> generate(const Shape& shape, const Scalar& h, const Scalar& k, const Scalar& max_distance) {
            std::vector<node_type> nodes;
            const Scalar jump = Scalar(1.0 / double(k));
            const Scalar circle = Scalar(2.0 * M_PI);

            // the node straight below the camera, linked to evenly spaced nodes of the first ring
            node_type origin{};
            origin.ray = vec3<Scalar>{{Scalar(0.0), Scalar(0.0), -Scalar(1.0)}};
            const int first_ring = int(std::ceil((k * circle) / shape.theta(jump, h)));
            const Scalar first_step = Scalar(first_ring) / Scalar(N_NEIGHBOURS);
            for (unsigned int i = 0; i < unsigned(N_NEIGHBOURS); ++i) origin.neighbours[i] = int(i * first_step) + 1;
            nodes.push_back(origin);

            int ring_start = 1;
            for (int ring = 1; h * std::tan(shape.phi(ring * jump, h)) < max_distance; ++ring) {
                const Scalar n_prev = (ring - 1) * jump;
                const Scalar n_cur = ring * jump;
                const Scalar n_next = (ring + 1) * jump;
                const Scalar size_prev = ring == 1 ? Scalar(1.0) : k * circle / shape.theta(n_prev, h);
                const Scalar size_cur = k * circle / shape.theta(n_cur, h);
                const Scalar size_next = k * circle / shape.theta(n_next, h);
                // spread the rounded-up number of nodes evenly around the ring
                const Scalar m_step = size_cur / (k * std::ceil(size_cur));

                ring_start = int(nodes.size());
                const int count_prev = int(std::ceil(size_prev)), count = int(std::ceil(size_cur)),
                          count_next = int(std::ceil(size_next));
                for (int j = 0; j < count; ++j) {
                    node_type node{};
                    node.ray = map(shape, h, vec2<Scalar>{{n_cur, j * m_step}});
                    const std::array<int, N_NEIGHBOURS> rel = neighbours(j, count_prev, count, count_next);
                    for (int t = 0; t < N_NEIGHBOURS; ++t) node.neighbours[t] = ring_start + rel[t];
                    nodes.push_back(node);
                }
            }

            // links past the last ring (and those of a lone origin) become "no neighbour" = nodes.size()
            const int total = int(nodes.size());
            for (int i = ring_start - 1; i < total; ++i)
                for (int& n : nodes[i].neighbours) n = std::min(n, total);
            return nodes;
        }
    };

}  // namespace model
}  // namespace visualmesh

#endif  // VISUALMESH_MODEL_RING6_HPP

/*
 * Mesh<Scalar, Model>: a Visual Mesh for one camera height - nodes in cone-tree order plus the tree that
 * answers "which index ranges can be on screen" (interface of reference mesh.hpp:56-609: constructor
 * :424-467, lookup :499-595, public members h, max_distance, nodes).
 *
 * Generation and lookup stay on the host. The HIP engine uploads `nodes` once per mesh and receives the
 * lookup ranges per frame.
 */
#ifndef VISUALMESH_MESH_HPP
#define VISUALMESH_MESH_HPP

#include <type_traits>
#include <utility>
#include <vector>

#include "detail/cone_tree.hpp"
#include "types.hpp"

namespace visualmesh {

template <typename Scalar, template <typename> class Model>
class Mesh {

public:
    static constexpr int N_NEIGHBOURS = Model<Scalar>::N_NEIGHBOURS;
    typedef Node<Scalar, N_NEIGHBOURS> node_type;

    /**
     * @param shape         object the mesh is sized for (Sphere, Circle)
     * @param h             height of the camera above the observation plane
     * @param k             number of mesh intersections per object
     * @param max_distance  how far along the plane the mesh reaches
     */
    template <typename Shape>
    Mesh(const Shape& shape, const Scalar& h, const Scalar& k, const Scalar& max_distance)
      : h(h), max_distance(max_distance) {
        std::vector<node_type> generated = Model<Scalar>::generate(shape, h, k, max_distance);
        const int n = int(generated.size());
        std::vector<vec3<Scalar>> rays(n);
        for (int i = 0; i < n; ++i) rays[i] = generated[i].ray;

        const std::vector<int> order = tree_.build(rays);

        // generation index -> sorted position; "no neighbour" (n) maps to itself
        std::vector<int> position(size_t(n) + 1);
        position[n] = n;
        for (int i = 0; i < n; ++i) position[order[i]] = i;
        nodes.resize(n);
        for (int i = 0; i < n; ++i) {
            nodes[i].ray = generated[order[i]].ray;
            for (int t = 0; t < N_NEIGHBOURS; ++t) nodes[i].neighbours[t] = position[generated[order[i]].neighbours[t]];
        }
    }

    /// A mesh of another scalar type converted to this one (reference mesh.hpp:476-488): same nodes in the same order with
    /// their unit vectors converted value by value, same neighbours, same tree with converted cones. Note that this is
    /// not the mesh that generating in this scalar type would give (ring sizes come from ceil() of quotients in Scalar).
    template <typename U>
    Mesh(const Mesh<U, Model>& other)
      : h(static_cast<Scalar>(other.h)), max_distance(static_cast<Scalar>(other.max_distance)), tree_(other.tree()) {
        nodes.reserve(other.nodes.size());
        for (const auto& n : other.nodes) {
            node_type mine;
            mine.ray = vec3<Scalar>{{static_cast<Scalar>(n.ray[0]), static_cast<Scalar>(n.ray[1]), static_cast<Scalar>(n.ray[2])}};
            for (int t = 0; t < N_NEIGHBOURS; ++t) mine.neighbours[t] = n.neighbours[t];
            nodes.push_back(mine);
        }
    }

    /// Index ranges [first, last) of nodes that may be on screen, ascending and disjoint.
    std::vector<std::pair<int, int>> lookup(const mat4<Scalar>& Hoc, const Lens<Scalar>& lens) const {
        return tree_.visible_ranges([this](int i) -> const vec3<Scalar>& { return nodes[i].ray; }, Hoc, lens);
    }

    /// The cone tree behind lookup(), for walks that run elsewhere (the HIP engine's lookup on the device)
#define VISUALMESH_MESH_HAS_CONE_TREE 1
    const detail::ConeTreeT<Scalar>& tree() const { return tree_; }

    Scalar h;                      ///< camera height this mesh was generated for
    Scalar max_distance;           ///< reach of the mesh
    std::vector<node_type> nodes;  ///< nodes in cone-tree order

private:
    detail::ConeTreeT<Scalar> tree_;
};

}  // namespace visualmesh

#endif  // VISUALMESH_MESH_HPP

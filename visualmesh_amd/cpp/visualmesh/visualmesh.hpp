/*
 * VisualMesh<Scalar, Model>: meshes for a range of camera heights, spaced so that the intersection count
 * k drifts by at most max_error between neighbouring heights, and the pick of the closest one
 * (interface of reference visualmesh.hpp:41-161: constructor :64-96, height() :122-135).
 */
#ifndef VISUALMESH_VISUALMESH_HPP
#define VISUALMESH_VISUALMESH_HPP

#include <cmath>
#include <iterator>
#include <map>
#include <utility>
#include <vector>

#include "mesh.hpp"
#include "model/ring6.hpp"

namespace visualmesh {

template <typename Scalar = float, template <typename> class Model = model::Ring6>
class VisualMesh {
public:
    VisualMesh() = default;

    template <typename Shape>
    explicit VisualMesh(const Shape& shape, const Scalar& min_height, const Scalar& max_height, const Scalar& k,
                        const Scalar& max_error, const Scalar& max_distance) {
        auto add = [&](const Scalar& h) {
            if (luts.find(h) == luts.end()) luts.emplace(h, Mesh<Scalar, Model>(shape, h, k, max_distance));
        };
        add(min_height);
        add(max_height);
        // halve every height interval whose ends disagree with its middle by more than max_error
        std::vector<vec2<Scalar>> todo(1, vec2<Scalar>{{min_height, max_height}});
        while (!todo.empty()) {
            const vec2<Scalar> span = todo.back();
            todo.pop_back();
            const Scalar h = (span[0] + span[1]) / 2;
            const Scalar low_error = std::abs(k - k * shape.k(span[0], h));
            const Scalar high_error = std::abs(k - k * shape.k(span[1], h));
            if (low_error > max_error || high_error > max_error) {
                add(h);
                todo.push_back(vec2<Scalar>{{span[0], h}});
                todo.push_back(vec2<Scalar>{{h, span[1]}});
            }
        }
    }

    /// A VisualMesh of another scalar type converted to this one (reference visualmesh.hpp:104-110): every height and
    /// every mesh converted (Mesh's converting constructor).
    template <typename U>
    VisualMesh(const VisualMesh<U, Model>& other) {
        for (const auto& entry : other.meshes()) luts.emplace(static_cast<Scalar>(entry.first), Mesh<Scalar, Model>(entry.second));
    }

    /// The mesh generated for the height closest to `height`; ties go to the lower mesh.
    const Mesh<Scalar, Model>& height(const Scalar& height) const {
        auto it = luts.lower_bound(height);
        if (it == luts.begin()) return it->second;
        if (it == luts.end()) return luts.rbegin()->second;
        auto below = std::prev(it);
        return std::abs(it->first - height) < std::abs(below->first - height) ? it->second : below->second;
    }

    /// All meshes by height (an addition to the reference interface: engines use it to pre-upload).
    const std::map<Scalar, const Mesh<Scalar, Model>>& meshes() const { return luts; }

private:
    std::map<Scalar, const Mesh<Scalar, Model>> luts;
};

}  // namespace visualmesh

#endif  // VISUALMESH_VISUALMESH_HPP

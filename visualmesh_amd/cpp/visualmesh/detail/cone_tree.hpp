/*
 * Binary partition of a mesh's unit vectors into nested bounding cones, and the walk that turns a camera
 * pose and lens into the index ranges that may be on screen.
 *
 * The engine contract is "same ranges as the reference": the ranges are a heuristic, not the exact
 * visible set, and the visible-node indices the engines return are only bit-identical if the node order
 * and the ranges are. This file therefore follows the reference's decisions exactly -
 *   bounding cone (incremental, order dependent)      reference mesh.hpp:96-118
 *   tree construction (root split on the sign of y, then mean-phi / mean-theta splits with
 *   std::partition, leaves of <= 8 nodes std::sort-ed)  reference mesh.hpp:135-248
 *   pre-shuffle with a fixed xorshift seed             reference mesh.hpp:433-442
 *   screen edge cones / planes                         reference mesh.hpp:265-349
 *   cone-versus-screen test                            reference mesh.hpp:362-406
 *   the stack walk                                     reference mesh.hpp:499-595
 * - and uses the same standard algorithms on the same iterator type (std::vector<int>::iterator), because
 * the permutation std::partition produces is part of the result.
 */
#ifndef VISUALMESH_DETAIL_CONE_TREE_HPP
#define VISUALMESH_DETAIL_CONE_TREE_HPP

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <limits>
#include <numeric>
#include <stdexcept>
#include <utility>
#include <vector>

#include "exact_math.hpp"
#include "lens_math.hpp"

namespace visualmesh {
namespace detail {

    template <typename T>
    class ConeTreeT {
    public:
        struct Element {
            int first, last;  ///< node range [first, last) in sorted order
            int child[2];     ///< -1, -1 for a leaf
            ConeT<T> cone;
        };

        /// Builds the tree over `rays` (generation order) and returns the sorted order:
        /// order[new_position] = generation index.
        std::vector<int> build(const std::vector<vec3<T>>& rays) {
            rays_ = &rays;
            std::vector<int> order(rays.size());
            std::iota(order.begin(), order.end(), 0);
            // light shuffle so the incremental bounding cone stays near linear
            uint32_t x = 0x4d657368;
            for (int i = int(order.size()) - 1; i > 0; i -= 5) {
                x ^= x << 13;
                x ^= x >> 17;
                x ^= x << 5;
                std::swap(order[i], order[x % i]);
            }
            elements_.clear();
            elements_.reserve(rays.size() * 2);
            split(order.begin(), order.end(), 0);
            rays_ = nullptr;
            return order;
        }

        const std::vector<Element>& elements() const { return elements_; }

        ConeTreeT() = default;
        /// The same tree over another scalar type: ranges and children as they are, every cone's axis, cosine and sine
        /// converted value by value (what reference mesh.hpp:476-488 does with its bsp entries).
        template <typename U>
        explicit ConeTreeT(const ConeTreeT<U>& other) {
            elements_.reserve(other.elements().size());
            for (const typename ConeTreeT<U>::Element& e : other.elements()) {
                Element mine;
                mine.first = e.first, mine.last = e.last;
                mine.child[0] = e.child[0], mine.child[1] = e.child[1];
                mine.cone.axis = vec3<T>{{static_cast<T>(e.cone.axis[0]), static_cast<T>(e.cone.axis[1]), static_cast<T>(e.cone.axis[2])}};
                mine.cone.c = static_cast<T>(e.cone.c);
                mine.cone.s = static_cast<T>(e.cone.s);
                elements_.push_back(mine);
            }
        }

        /// What a walk of the tree compares an element against, for one camera pose: the field-of-view cone and the
        /// four cones (or planes) along the screen edges. visible_ranges() works these out for itself; a walk that
        /// runs elsewhere (on the device) is handed them.
        struct Parameters {
            T cos_half_fov, sin_half_fov;
            ConeT<T> edges[4];
        };
        static Parameters lookup_parameters(const mat4<T>& Hoc, const Lens<T>& lens) {
            Parameters p;
            p.cos_half_fov = std::cos(lens.fov * T(0.5));
            p.sin_half_fov = std::sin(lens.fov * T(0.5));
            screen_edges(Hoc, lens, p.edges);
            return p;
        }

        /// On-screen candidate ranges. ray_at(i) returns the unit vector of node i in sorted order.
        template <typename RayAt>
        std::vector<std::pair<int, int>> visible_ranges(const RayAt& ray_at, const mat4<T>& Hoc, const Lens<T>& lens) const {
            const T cos_half_fov = std::cos(lens.fov * T(0.5));
            const T sin_half_fov = std::sin(lens.fov * T(0.5));
            const mat3<T> Rco = rotation_co(Hoc);
            const vec3<T> optical_axis = Rco[0];
            ConeT<T> edges[4];
            screen_edges(Hoc, lens, edges);

            std::vector<std::pair<int, int>> ranges;
            if (elements_.empty()) return ranges;
            std::vector<int> todo(1, 0);
            bool open = false;
            int open_first = 0, open_last = 0;
            auto close = [&]() {
                if (open) {
                    ranges.emplace_back(open_first, open_last);
                    open = false;
                }
            };
            while (!todo.empty()) {
                const Element& e = elements_[todo.back()];
                todo.pop_back();

                // field-of-view cone first: cos(a -/+ b) by the compound angle formula
                const T along = dot(optical_axis, e.cone.axis);
                bool outside = along < cos_half_fov * e.cone.c - sin_half_fov * e.cone.s;
                bool inside = along > cos_half_fov * e.cone.c + sin_half_fov * e.cone.s;
                if (!outside && inside) cone_on_screen(Rco, e.cone, lens, edges, inside, outside);

                if (inside) {
                    if (!open) {
                        open_first = e.first;
                        open = true;
                    }
                    open_last = e.last;
                }
                else if (outside) {
                    close();
                }
                else if (e.child[0] < 0) {
                    for (int i = e.first; i < e.last; ++i) {
                        const vec3<T> ray = ray_at(i);
                        const vec2<T> px = project(apply(Rco, ray), lens);
                        const bool on_screen = dot(optical_axis, ray) > cos_half_fov && 0 <= px[0] && px[0] + 1 <= lens.dimensions[0]
                                               && 0 <= px[1] && px[1] + 1 <= lens.dimensions[1];
                        if (on_screen) {
                            if (!open) {
                                open_first = i;
                                open = true;
                            }
                            open_last = i + 1;
                        }
                        else {
                            close();
                        }
                    }
                }
                else {
                    todo.push_back(e.child[1]);
                    todo.push_back(e.child[0]);
                }
            }
            close();
            return ranges;
        }

    private:
        typedef std::vector<int>::iterator Iter;

        ConeT<T> enclose(Iter begin, Iter end) const {
            const std::vector<vec3<T>>& R = *rays_;
            ConeT<T> k = cone_through<T>();
            for (Iter a = begin; a < end; ++a) {
                if (!(dot(k.axis, R[*a]) < k.c)) continue;
                k = cone_through(R[*a]);
                for (Iter b = begin; b < a; ++b) {
                    if (!(dot(k.axis, R[*b]) < k.c)) continue;
                    k = cone_through(R[*a], R[*b]);
                    for (Iter c = begin; c < b; ++c) {
                        if (dot(k.axis, R[*c]) < k.c) k = cone_through(R[*a], R[*b], R[*c]);
                    }
                }
            }
            return with_sine(k);
        }

        int split(Iter begin, Iter end, int offset) {
            const std::vector<vec3<T>>& R = *rays_;
            const int count = int(std::distance(begin, end));
            if (count == 0) throw std::runtime_error("We tried to make a tree with no nodes");
            const int leaf_size = 8;

            if (count <= leaf_size) {
                const int id = int(elements_.size());
                elements_.push_back(Element{offset, offset + count, {-1, -1}, enclose(begin, end)});
                std::sort(begin, end);  // generation order inside a leaf
                return id;
            }

            if (elements_.empty()) {
                // root: the cone around straight-down that reaches the highest node; children = sign of y
                Iter top = std::max_element(begin, end, [&R](const int& a, const int& b) { return R[a][2] < R[b][2]; });
                const T c = -R[*top][2];
                const T s = std::sqrt(1 - c * c);
                Iter mid = std::partition(begin, end, [&R](const int& a) { return R[a][1] > 0; });
                elements_.push_back(Element{offset, count, {-1, -1}, ConeT<T>{vec3<T>{{0, 0, -1}}, c, s}});
                const int left = split(begin, mid, 0);
                const int right = split(mid, end, int(std::distance(begin, mid)));
                elements_[0].child[0] = left;
                elements_[0].child[1] = right;
                return 0;
            }

            const ConeT<T> cone = enclose(begin, end);

            // extents of z ("phi") and of x / sqrt(1 - z^2) ("theta"); split the wider one at its mean
            T z_min = std::numeric_limits<T>::max(), z_max = std::numeric_limits<T>::lowest();
            T t_min = std::numeric_limits<T>::max(), t_max = std::numeric_limits<T>::lowest();
            T z_sum = 0, t_sum = 0;
            int z_count = 0, t_count = 0;
            for (Iter it = begin; it != end; ++it) {
                const vec3<T>& ray = R[*it];
                const T z = ray[2];
                const T t = ray[0] / std::sqrt(1 - ray[2] * ray[2]);
                z_min = std::min(z_min, z);
                z_max = std::max(z_max, z);
                z_sum += z;
                z_count += 1;
                if (std::isfinite(t)) {
                    t_min = std::min(t_min, t);
                    t_max = std::max(t_max, t);
                    t_sum += t;
                    t_count += 1;
                }
            }
            const T z_split = z_sum / z_count;
            const T t_split = t_sum / t_count;
            Iter mid = z_max - z_min > t_max - t_min
                         ? std::partition(begin, end, [&R, &z_split](const int& a) { return R[a][2] > z_split; })
                         : std::partition(begin, end, [&R, &t_split](const int& a) {
                               return R[a][0] / std::sqrt(1 - R[a][2] * R[a][2]) < t_split;  // NaN (the origin) goes right
                           });

            const int id = int(elements_.size());
            elements_.push_back(Element{offset, offset + count, {-1, -1}, cone});
            const int left = split(begin, mid, offset);
            const int right = split(mid, end, offset + int(std::distance(begin, mid)));
            elements_[id].child[0] = left;
            elements_[id].child[1] = right;
            return id;
        }

        /// Four cones (fisheye) or planes (rectilinear) hugging the image edges, in observation-plane space.
        static void screen_edges(const mat4<T>& Hoc, const Lens<T>& lens, ConeT<T> (&edges)[4]) {
            const mat3<T> Roc = rotation_oc(Hoc);
            // one pixel inside the border
            const vec2<T> far{{T(lens.dimensions[0]) - T(1.0), T(lens.dimensions[1]) - T(1.0)}};
            const vec3<T> corner[4] = {
              apply(Roc, unproject(vec2<T>{{1, 1}}, lens)),
              apply(Roc, unproject(vec2<T>{{far[0], 1}}, lens)),
              apply(Roc, unproject(vec2<T>{{far[0], far[1]}}, lens)),
              apply(Roc, unproject(vec2<T>{{1, far[1]}}, lens)),
            };
            switch (lens.projection) {
                case RECTILINEAR:
                    for (int i = 0; i < 4; ++i) edges[i] = ConeT<T>{unit(cross(corner[(i + 1) & 3], corner[i])), 0, 1};
                    return;
                case EQUIDISTANT:
                case EQUISOLID: {
                    const vec2<T> mid{{far[0] * T(0.5) + lens.centre[0], far[1] * T(0.5) + lens.centre[1]}};
                    const vec3<T> edge_mid[4] = {
                      apply(Roc, unproject(vec2<T>{{mid[0], 1}}, lens)),
                      apply(Roc, unproject(vec2<T>{{far[0], mid[1]}}, lens)),
                      apply(Roc, unproject(vec2<T>{{mid[0], far[1]}}, lens)),
                      apply(Roc, unproject(vec2<T>{{1, mid[1]}}, lens)),
                    };
                    for (int i = 0; i < 4; ++i) edges[i] = with_sine(cone_through(corner[(i + 1) & 3], edge_mid[i], corner[i]));
                    return;
                }
                default: throw std::runtime_error("Unknown lens type");
            }
        }

        static void cone_on_screen(const mat3<T>& Rco, const ConeT<T>& cone, const Lens<T>& lens, const ConeT<T> (&edges)[4],
                                   bool& inside, bool& outside) {
            const vec2<T> px = project(apply(Rco, cone.axis), lens);
            const bool axis_on_screen =
              0 <= px[0] && px[0] + 1 <= lens.dimensions[0] && 0 <= px[1] && px[1] + 1 <= lens.dimensions[1];
            T along[4];
            bool beyond = false;
            for (int i = 0; i < 4; ++i) {
                along[i] = dot(cone.axis, edges[i].axis);
                beyond = beyond || along[i] > edges[i].c * cone.c + edges[i].s * cone.s;
            }
            if (!axis_on_screen && beyond) {
                inside = false;
                outside = true;
                return;
            }
            bool clear = true;
            for (int i = 0; i < 4; ++i) clear = clear && along[i] < edges[i].c * cone.c - edges[i].s * cone.s;
            inside = axis_on_screen && clear;
            outside = false;
        }

        std::vector<Element> elements_;
        const std::vector<vec3<T>>* rays_ = nullptr;
    };

    typedef ConeTreeT<float> ConeTree;

}  // namespace detail
}  // namespace visualmesh

#endif  // VISUALMESH_DETAIL_CONE_TREE_HPP

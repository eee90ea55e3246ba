/* Meshes and VisualMeshes converted between scalar types (reference mesh.hpp:476-488, visualmesh.hpp:104-110). The same
 * source is compiled once against this repository's host headers and once against the reference's; tests/test_abi.py
 * compares what the two programs print: node counts, digests of rays and neighbours, and the lookup ranges of the
 * converted meshes. Only the reference's public interface is used. */
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <limits>     // the reference's headers use these two without including them
#include <stdexcept>
#include <utility>
#include <vector>

#include "visualmesh/geometry/Sphere.hpp"
#include "visualmesh/lens.hpp"
#include "visualmesh/mesh.hpp"
#include "visualmesh/model/ring6.hpp"
#include "visualmesh/visualmesh.hpp"

using visualmesh::model::Ring6;

static uint64_t fnv(uint64_t h, const void* data, size_t n) {
    const unsigned char* p = static_cast<const unsigned char*>(data);
    for (size_t i = 0; i < n; ++i) h = (h ^ p[i]) * 1099511628211ull;
    return h;
}

template <typename Scalar>
static void describe(const char* label, const visualmesh::Mesh<Scalar, Ring6>& mesh) {
    uint64_t rays = 14695981039346656037ull, neighbours = rays;
    for (const auto& n : mesh.nodes) {
        for (int c = 0; c < 3; ++c) rays = fnv(rays, &n.ray[c], sizeof(Scalar));
        for (int t = 0; t < 6; ++t) neighbours = fnv(neighbours, &n.neighbours[t], sizeof(int));
    }
    std::printf("%s nodes %zu h %.17g max_distance %.17g rays %016llx neighbours %016llx\n", label, mesh.nodes.size(), double(mesh.h),
                double(mesh.max_distance), (unsigned long long) rays, (unsigned long long) neighbours);
    visualmesh::mat4<Scalar> Hoc = {{{{Scalar(0.8660254), 0, Scalar(0.5), 0}}, {{0, 1, 0, 0}}, {{Scalar(-0.5), 0, Scalar(0.8660254), Scalar(1.0)}}, {{0, 0, 0, 1}}}};
    for (int projection = 0; projection < 2; ++projection) {
        visualmesh::Lens<Scalar> lens;
        lens.dimensions = {{640, 480}};
        lens.projection = projection == 0 ? visualmesh::EQUISOLID : visualmesh::RECTILINEAR;
        lens.focal_length = projection == 0 ? Scalar(210) : Scalar(400);
        lens.centre = {{0, 0}};
        lens.k = {{0, 0}};
        lens.fov = projection == 0 ? Scalar(3.14159265) : Scalar(1.4);
        const std::vector<std::pair<int, int>> ranges = mesh.lookup(Hoc, lens);
        std::printf("%s lens %d ranges %zu:", label, projection, ranges.size());
        for (const auto& r : ranges) std::printf(" %d-%d", r.first, r.second);
        std::printf("\n");
    }
}

int main() {
    const visualmesh::geometry::Sphere<double> ball(0.0949);
    const visualmesh::geometry::Sphere<float> ball_f(0.0949f);
    const visualmesh::Mesh<double, Ring6> generated_in_double(ball, 1.0, 4.0, 6.0);
    const visualmesh::Mesh<float, Ring6> generated_in_float(ball_f, 1.0f, 4.0f, 6.0f);
    const visualmesh::Mesh<float, Ring6> to_float(generated_in_double);
    const visualmesh::Mesh<double, Ring6> to_double(generated_in_float);
    describe("double", generated_in_double);
    describe("double->float", to_float);
    describe("float", generated_in_float);
    describe("float->double", to_double);
    const visualmesh::VisualMesh<double, Ring6> heights(ball, 0.8, 1.2, 4.0, 0.5, 6.0);
    const visualmesh::VisualMesh<float, Ring6> heights_f(heights);
    for (float h : {0.7f, 0.85f, 0.95f, 1.0f, 1.1f, 1.3f}) {
        char label[64];
        std::snprintf(label, sizeof label, "heights->float at %.2f", double(h));
        describe(label, heights_f.height(h));
    }
    return 0;
}

/* The reference engines' interface on the HIP engine, compiled against the REFERENCE's own headers (its include
 * directory comes first on the command line, so visualmesh/mesh.hpp, visualmesh.hpp, lens.hpp ... are the reference's and
 * only visualmesh/engine/hip/engine.hpp is this repository's): what a maintainer gets after dropping engine.hpp into
 * cpp/visualmesh/engine/hip/. tests/test_abi.py compiles it (syntax and templates only) where the reference tree is
 * mounted. */
#include <cstdint>
#include <limits>     // the reference's headers use these two without including them
#include <stdexcept>
#include <vector>

#include "visualmesh/engine/hip/engine.hpp"
#include "visualmesh/geometry/Sphere.hpp"
#include "visualmesh/mesh.hpp"
#include "visualmesh/model/ring6.hpp"
#include "visualmesh/utility/fourcc.hpp"
#include "visualmesh/visualmesh.hpp"

/* the same calls for both Scalars the reference's engines are instantiated with (engine/cpu/engine.hpp:49-50) */
template <typename Scalar>
int use_engine() {
    visualmesh::geometry::Sphere<Scalar> shape(Scalar(0.0949));
    visualmesh::Mesh<Scalar, visualmesh::model::Ring6> mesh(shape, Scalar(1.2), Scalar(6.0), Scalar(5.0));
    visualmesh::VisualMesh<Scalar, visualmesh::model::Ring6> heights(shape, Scalar(0.8), Scalar(1.5), Scalar(6.0), Scalar(0.5), Scalar(5.0));
    visualmesh::NetworkStructure<Scalar> network;
    visualmesh::engine::hip::Engine<Scalar> engine(network);
    visualmesh::mat4<Scalar> Hoc = {{{{1, 0, 0, 0}}, {{0, 1, 0, 0}}, {{0, 0, 1, Scalar(1.2)}}, {{0, 0, 0, 1}}}};
    visualmesh::Lens<Scalar> lens;
    lens.dimensions = {{1280, 1024}};
    lens.projection = visualmesh::EQUISOLID;
    lens.focal_length = 420;
    lens.centre = {{0, 0}};
    lens.k = {{0, 0}};
    lens.fov = Scalar(3.14159265);
    std::vector<uint8_t> image(1280 * 1024 * 4);
    visualmesh::ProjectedMesh<Scalar, visualmesh::model::Ring6<Scalar>::N_NEIGHBOURS> projected = engine(mesh, Hoc, lens);
    auto projected_too = engine.project(mesh, Hoc, lens);
    visualmesh::ClassifiedMesh<Scalar, visualmesh::model::Ring6<Scalar>::N_NEIGHBOURS> classified =
      engine(mesh, Hoc, lens, image.data(), visualmesh::fourcc("RGBA"));
    auto by_height = engine(heights, Hoc, lens, image.data(), visualmesh::fourcc("RGBA"));
    auto projected_by_height = engine(heights, Hoc, lens);
    engine.clear_cache();
    return int(projected.global_indices.size() + projected_too.global_indices.size() + classified.global_indices.size()
               + by_height.global_indices.size() + projected_by_height.global_indices.size());
}

int main() { return use_engine<float>() + use_engine<double>(); }

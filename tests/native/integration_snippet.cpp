/* The call sites a user of the reference writes, with the engine type changed to the HIP engine: this file must
 * compile against the host headers alone (any C++14 compiler, no HIP headers), and link against
 * libvisualmesh_hip.so. tests/test_abi.py compiles and links it; tests/test_gpu_edges.py also runs it. */
#include <cstdint>
#include <cstdio>
#include <vector>

#include "visualmesh/engine/hip/engine.hpp"
#include "visualmesh/geometry/Sphere.hpp"
#include "visualmesh/mesh.hpp"
#include "visualmesh/model/ring6.hpp"
#include "visualmesh/utility/fourcc.hpp"
#include "visualmesh/visualmesh.hpp"

int main() {
    using Scalar = float;
    visualmesh::geometry::Sphere<Scalar> shape(0.0949f);
    visualmesh::Mesh<Scalar, visualmesh::model::Ring6> mesh(shape, 1.2f, 6.0f, 5.0f);
    visualmesh::VisualMesh<Scalar, visualmesh::model::Ring6> heights(shape, 0.8f, 1.5f, 6.0f, 0.5f, 5.0f);
    visualmesh::NetworkStructure<Scalar> network;  // as load_model() returns it
    visualmesh::engine::hip::Engine<Scalar> engine(network);

    visualmesh::mat4<Scalar> Hoc = {{{{1, 0, 0, 0}}, {{0, 1, 0, 0}}, {{0, 0, 1, 1.2f}}, {{0, 0, 0, 1}}}};
    visualmesh::Lens<Scalar> lens;
    lens.dimensions = {{1280, 1024}};
    lens.projection = visualmesh::EQUISOLID;
    lens.focal_length = 420;
    lens.centre = {{0, 0}};
    lens.k = {{0, 0}};
    lens.fov = 3.14159265f;
    std::vector<uint8_t> image(1280 * 1024 * 4);

    // the reference engines' interface
    auto projected = engine(mesh, Hoc, lens);
    auto projected_too = engine.project(mesh, Hoc, lens);
    auto classified = engine(mesh, Hoc, lens, image.data(), visualmesh::fourcc("RGBA"));
    auto by_height = engine(heights, Hoc, lens, image.data(), visualmesh::fourcc("RGBA"));
    engine.clear_cache();

    // what the HIP engine adds
    typedef visualmesh::engine::hip::Engine<Scalar>::Frame<visualmesh::model::Ring6> Frame;
    std::vector<Frame> frames(2, Frame{&mesh, Hoc, lens, image.data(), visualmesh::fourcc("RGBA")});
    auto results = engine.classify(frames);
    engine.stage(frames);
    engine.run();
    auto detections = engine.detect(0, 0.5f);
    auto graph = engine.lookup_graph<visualmesh::model::Ring6>(visualmesh::engine::hip::Engine<Scalar>::SAME);
    engine.run_async();
    engine.wait();
    auto fetched = engine.fetch<visualmesh::model::Ring6>();
    // results into arrays of the caller's (page-locked ones make the copies asynchronous), in one call or in two halves
    const std::vector<int32_t> visible = engine.visible_counts();
    const int classes = 4;  // an empty network returns the four sampled channels
    std::vector<std::vector<float>> px(frames.size()), cls(frames.size());
    std::vector<std::vector<int32_t>> gidx(frames.size()), nb(frames.size());
    std::vector<vmhip_result> into(frames.size());
    for (size_t i = 0; i < frames.size(); ++i) {
        px[i].resize(size_t(visible[i]) * 2), gidx[i].resize(visible[i]), nb[i].resize((size_t(visible[i]) + 1) * 6),
          cls[i].resize((size_t(visible[i]) + 1) * classes);
        into[i] = vmhip_result{visible[i], 0, px[i].data(), gidx[i].data(), nb[i].data(), cls[i].data()};
    }
    engine.fetch_into(into);
    const bool into_same = gidx[1] == fetched[1].global_indices;
    engine.fetch_into_async(into);
    engine.fetch_wait();
    engine.set_device_lookup(true);
    engine.stage(frames);
    engine.run();
    const bool device_lookup_same = engine.visible_counts() == visible;
    engine.set_device_lookup(false);
    // an engine moved while a batch is staged: the staged frames' mesh stays pinned in the moved-to engine's cache (the
    // limit below is smaller than any mesh, so everything that is not pinned goes when another mesh comes in), and the
    // cache's accounting travels along
    engine.set_cache_limit(1);
    engine.stage(frames);
    const size_t bytes_before = engine.cache_bytes();
    visualmesh::engine::hip::Engine<Scalar> moved(std::move(engine));
    const bool accounting_moved = moved.cache_bytes() == bytes_before && bytes_before > 0 && engine.cache_bytes() == 0;
    auto other_mesh = moved(heights, Hoc, lens);  // uploads the height's mesh and trims the cache
    moved.run();                                  // runs on the staged mesh, which must still be on the device
    const bool moved_same = moved.visible_counts() == visible && moved.cached_meshes() >= 1 && accounting_moved
                            && other_mesh.global_indices == by_height.global_indices;
    std::printf("projected %zu %zu classified %zu by_height %zu batch %zu %zu detections %zu graph %zu fetched %zu\n",
                projected.global_indices.size(), projected_too.global_indices.size(), classified.global_indices.size(),
                by_height.global_indices.size(), results.size(), results[1].global_indices.size(), detections.size(),
                graph[0].vectors.size(), fetched[0].global_indices.size());
    const bool same = projected.global_indices == projected_too.global_indices && projected.global_indices == classified.global_indices
                      && classified.global_indices == results[1].global_indices && classified.global_indices == fetched[0].global_indices
                      && graph[0].vectors.size() >= projected.global_indices.size() && !projected.global_indices.empty() && into_same
                      && device_lookup_same && moved_same;
    std::printf(same ? "ok\n" : "MISMATCH\n");
    return same ? 0 : 1;
}

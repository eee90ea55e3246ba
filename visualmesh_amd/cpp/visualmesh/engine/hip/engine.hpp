/*
 * visualmesh::engine::hip::Engine - the Visual Mesh engine for AMD MI355X (gfx950).
 *
 * Same interface as the reference's engines (reference engine/cpu/engine.hpp:49-306,
 * engine/opencl/engine.hpp:172-572):
 *
 *     Engine(const NetworkStructure<Scalar>& structure = {});
 *     ProjectedMesh  engine(mesh, Hoc, lens);                    // also engine.project(mesh, Hoc, lens)
 *     ClassifiedMesh engine(mesh, Hoc, lens, image, format);
 *
 * with `mesh` either a Mesh<Scalar, Model> or a VisualMesh<Scalar, Model> (which picks the mesh for the
 * camera height Hoc[2][3]). In addition a batch of frames can be classified in one pass, either in one
 * call (classify(frames)) or staged (stage / run / fetch) to keep inputs resident on the device.
 *
 * This header is host C++14 and contains no device code: it runs Mesh::lookup on the host, flattens the
 * STL types and calls the C ABI of libvisualmesh_hip.so (include/visualmesh_hip.h). It only uses
 * `mesh.nodes` and `mesh.lookup(Hoc, lens)`, so it works with any Mesh type that has them.
 *
 * Results are those of the reference CPU engine on a fresh engine object: visible-node indices and the
 * neighbourhood table bit for bit, pixel coordinates to the last bits of acosf/sinf/tanf, class
 * probabilities to summation order.
 *
 * Errors: an unsupported fourcc or lens projection throws std::runtime_error with the reference's
 * message; any other failure throws std::system_error with hip_error_category(). An empty visible set is
 * not an error and returns a default-constructed result.
 *
 * Like the reference engines an Engine is not thread safe: use one engine per thread; meshes may be
 * shared.
 */
#ifndef VISUALMESH_ENGINE_HIP_ENGINE_HPP
#define VISUALMESH_ENGINE_HIP_ENGINE_HPP

/* VISUALMESH_DISABLE_HIP compiles the engine out, as VISUALMESH_DISABLE_OPENCL / _VULKAN do for the reference's engines
 * (reference cpp/CMakeLists.txt:30-53, example/benchmark.cpp:141-146): cmake/HipEngine.cmake defines it unless
 * BUILD_HIP_ENGINE is on. */
#if !defined(VISUALMESH_DISABLE_HIP)

#include <algorithm>
#include <cstdint>
#include <array>
#include <exception>
#include <thread>
#include <cstring>
#include <map>
#include <memory>
#include <stdexcept>
#include <string>
#include <system_error>
#include <type_traits>
#include <utility>
#include <vector>

#include "visualmesh/classified_mesh.hpp"
#include "visualmesh/lens.hpp"
#include "visualmesh/mesh.hpp"
#include "visualmesh/network_structure.hpp"
#include "visualmesh/projected_mesh.hpp"
#include "visualmesh/visualmesh.hpp"
#include "visualmesh_hip.h"

namespace visualmesh {
namespace engine {
    namespace hip {

        /// Error category for the status codes of libvisualmesh_hip.so.
        class error_category_t : public std::error_category {
        public:
            const char* name() const noexcept override { return "visualmesh_hip"; }
            std::string message(int code) const override {
                switch (code) {
                    case VMHIP_OK: return "success";
                    case VMHIP_ERR_HIP: return "HIP runtime failure";
                    case VMHIP_ERR_FORMAT: return "unsupported image format";
                    case VMHIP_ERR_LENS: return "unknown lens projection";
                    case VMHIP_ERR_ARGUMENT: return "invalid argument";
                    case VMHIP_ERR_CAPACITY: return "result buffer too small";
                    default: return "unknown error";
                }
            }
        };
        inline const std::error_category& hip_error_category() {
            static error_category_t instance;
            return instance;
        }
        inline void throw_on_error(int code) {
            if (code == VMHIP_OK) return;
            const std::string what = vmhip_last_error();
            if (code == VMHIP_ERR_FORMAT || code == VMHIP_ERR_LENS) throw std::runtime_error(what);
            throw std::system_error(code, hip_error_category(), what);
        }

        enum class Precision { FP32 = VMHIP_FP32, BF16 = VMHIP_BF16, FP64 = VMHIP_FP64, SPLIT = VMHIP_SPLIT };

        /// Engine<float> is the template below; Engine<double> is the specialisation at the end of this file.
        template <typename Scalar>
        class Engine {
            static_assert(std::is_same<Scalar, float>::value, "Scalar is float (this template) or double (the specialisation below)");

        public:
            /// One frame of a batch.
            template <template <typename> class Model>
            struct Frame {
                const Mesh<Scalar, Model>* mesh;
                mat4<Scalar> Hoc;
                Lens<Scalar> lens;
                const void* image;
                uint32_t format;
            };

            Engine(const NetworkStructure<Scalar>& structure = {}, Precision precision = Precision::FP32)
              : precision_(precision) {
                for (const auto& group : structure) {
                    group_sizes_.push_back(int32_t(group.size()));
                    for (const auto& layer : group) {
                        FlatLayer flat;
                        flat.n_in = int32_t(layer.weights.size());
                        flat.n_out = int32_t(layer.biases.size());
                        flat.activation = int32_t(layer.activation);
                        flat.weights.reserve(size_t(flat.n_in) * flat.n_out);
                        for (const auto& row : layer.weights) {
                            if (int32_t(row.size()) != flat.n_out) throw std::invalid_argument("ragged weight matrix");
                            flat.weights.insert(flat.weights.end(), row.begin(), row.end());
                        }
                        flat.biases = layer.biases;
                        layers_.push_back(std::move(flat));
                    }
                }
            }
            ~Engine() { release(); }
            Engine(const Engine&) = delete;
            Engine& operator=(const Engine&) = delete;
            Engine(Engine&& o) noexcept { *this = std::move(o); }
            Engine& operator=(Engine&& o) noexcept {
                if (this != &o) {
                    release();
                    precision_ = o.precision_;
                    group_sizes_ = std::move(o.group_sizes_);
                    layers_ = std::move(o.layers_);
                    engine_ = o.engine_;
                    engine_nn_ = o.engine_nn_;
                    batch_ = o.batch_;
                    meshes_ = std::move(o.meshes_);
                    staged_ = std::move(o.staged_);
                    /* the cache's book-keeping travels with the meshes: the staged frames' meshes are pinned by
                     * staged_since_, entries age against clock_, the byte count decides what is released */
                    clock_ = o.clock_;
                    staged_since_ = o.staged_since_;
                    staging_ = o.staging_;
                    device_lookup_ = o.device_lookup_;
                    cache_bytes_ = o.cache_bytes_;
                    cache_limit_ = o.cache_limit_;
                    o.engine_ = nullptr;
                    o.engine_nn_ = -1;
                    o.batch_ = nullptr;
                    o.meshes_.clear();
                    o.staged_.clear();
                    o.clock_ = 0, o.staged_since_ = 0, o.staging_ = false;
                    o.cache_bytes_ = 0;
                }
                return *this;
            }

            // ------------------------------------------------------------------ projection
            template <template <typename> class Model>
            ProjectedMesh<Scalar, Model<Scalar>::N_NEIGHBOURS> operator()(const Mesh<Scalar, Model>& mesh,
                                                                          const mat4<Scalar>& Hoc,
                                                                          const Lens<Scalar>& lens) const {
                constexpr int N = Model<Scalar>::N_NEIGHBOURS;
                FrameData fd;
                find_ranges(mesh, Hoc, lens, fd);
                describe(mesh, Hoc, lens, nullptr, 0, fd);
                ProjectedMesh<Scalar, N> out;
                /* nothing visible: no pixels, no indices, and the neighbourhood table is its null row alone, pointing
                 * at itself (reference engine/cpu/engine.hpp:127-143 with n_points = 0) */
                std::array<int, N> null_row;
                null_row.fill(0);
                if (fd.candidates == 0) {
                    out.neighbourhood.assign(1, null_row);
                    return out;
                }
                out.pixel_coordinates.resize(fd.candidates);
                out.global_indices.resize(fd.candidates);
                out.neighbourhood.resize(size_t(fd.candidates) + 1);
                vmhip_result r{};
                r.capacity = fd.candidates;
                r.pixel_coordinates = reinterpret_cast<float*>(out.pixel_coordinates.data());
                r.global_indices = out.global_indices.data();
                r.neighbourhood = reinterpret_cast<int32_t*>(out.neighbourhood.data());
                throw_on_error(vmhip_project(handle(N), &fd.frame, &r));
                if (r.n_visible == 0) {
                    ProjectedMesh<Scalar, N> none;
                    none.neighbourhood.assign(1, null_row);
                    return none;
                }
                out.pixel_coordinates.resize(r.n_visible);
                out.global_indices.resize(r.n_visible);
                out.neighbourhood.resize(size_t(r.n_visible) + 1);
                return out;
            }
            template <template <typename> class Model>
            ProjectedMesh<Scalar, Model<Scalar>::N_NEIGHBOURS> operator()(const VisualMesh<Scalar, Model>& mesh,
                                                                          const mat4<Scalar>& Hoc,
                                                                          const Lens<Scalar>& lens) const {
                return operator()(mesh.height(Hoc[2][3]), Hoc, lens);
            }
            template <typename AnyMesh>
            auto project(const AnyMesh& mesh, const mat4<Scalar>& Hoc, const Lens<Scalar>& lens) const
              -> decltype(this->operator()(mesh, Hoc, lens)) {
                return operator()(mesh, Hoc, lens);
            }

            // ------------------------------------------------------------------ classification
            template <template <typename> class Model>
            ClassifiedMesh<Scalar, Model<Scalar>::N_NEIGHBOURS> operator()(const Mesh<Scalar, Model>& mesh,
                                                                           const mat4<Scalar>& Hoc,
                                                                           const Lens<Scalar>& lens,
                                                                           const void* image,
                                                                           const uint32_t& format) const {
                std::vector<Frame<Model>> one(1, Frame<Model>{&mesh, Hoc, lens, image, format});
                return std::move(classify(one)[0]);
            }
            template <template <typename> class Model>
            ClassifiedMesh<Scalar, Model<Scalar>::N_NEIGHBOURS> operator()(const VisualMesh<Scalar, Model>& mesh,
                                                                           const mat4<Scalar>& Hoc,
                                                                           const Lens<Scalar>& lens,
                                                                           const void* image,
                                                                           const uint32_t& format) const {
                return operator()(mesh.height(Hoc[2][3]), Hoc, lens, image, format);
            }

            /// Classify a batch of independent frames in one pass over the device.
            template <template <typename> class Model>
            std::vector<ClassifiedMesh<Scalar, Model<Scalar>::N_NEIGHBOURS>> classify(const std::vector<Frame<Model>>& frames) const {
                stage(frames);
                run();
                return fetch<Model>();
            }

            /// Copy the frames' inputs to the device (images, poses, lenses, lookup ranges).
            template <template <typename> class Model>
            void stage(const std::vector<Frame<Model>>& frames) const {
                stage_frames(frames, true);
            }
            /// The same without waiting for the copies: they are queued ahead of the run and the call returns. The
            /// images must be page-locked (vmhip_host_alloc) and stay untouched until run() or wait() has returned.
            template <template <typename> class Model>
            void stage_async(const std::vector<Frame<Model>>& frames) const {
                stage_frames(frames, false);
            }

        private:
            template <template <typename> class Model>
            void stage_frames(const std::vector<Frame<Model>>& frames, bool wait_for_copies) const {
                constexpr int N = Model<Scalar>::N_NEIGHBOURS;
                staged_since_ = ++clock_;
                staged_.assign(frames.size(), FrameData());
                std::vector<vmhip_frame> flat(frames.size());
                staging_ = true;  // meshes described from here on belong to the staged batch
                try {
                    /* the lookups are independent of each other and of the device: a few threads share them (each takes
                     * ~80 us for a 1.2e5-node mesh), then the frames are described one by one (the mesh cache is not
                     * thread safe) */
                    const size_t n = frames.size();
                    for (size_t i = 0; i < n; ++i) staged_[i].lookup_on_device = device_lookup_;
                    const size_t workers = device_lookup_ ? 0 : std::min<size_t>(std::min<size_t>(n, 8), std::max(1u, std::thread::hardware_concurrency()));
                    std::vector<std::exception_ptr> failed(std::max<size_t>(workers, 1));
                    auto look_up = [&](size_t w) {
                        try {
                            for (size_t i = w; i < n; i += workers) find_ranges(*frames[i].mesh, frames[i].Hoc, frames[i].lens, staged_[i]);
                        } catch (...) {
                            failed[w] = std::current_exception();
                        }
                    };
                    std::vector<std::thread> pool;
                    for (size_t w = 1; w < workers; ++w) pool.emplace_back(look_up, w);
                    if (workers > 0) look_up(0);
                    for (auto& t : pool) t.join();
                    for (auto& e : failed)
                        if (e) std::rethrow_exception(e);
                    for (size_t i = 0; i < n; ++i) {
                        describe(*frames[i].mesh, frames[i].Hoc, frames[i].lens, frames[i].image, frames[i].format, staged_[i]);
                        flat[i] = staged_[i].frame;
                    }
                } catch (...) {
                    staging_ = false;
                    staged_.clear();
                    throw;
                }
                staging_ = false;
                vmhip_engine* e = handle(N);
                if (!batch_) throw_on_error(vmhip_batch_create(e, &batch_));
                if (!flat.empty())
                    throw_on_error(wait_for_copies ? vmhip_batch_stage(batch_, flat.data(), int32_t(flat.size()), 1)
                                                   : vmhip_batch_stage_async(batch_, flat.data(), int32_t(flat.size()), 1));
            }

        public:
            /// Run the staged frames on the device and wait; may be called repeatedly.
            void run() const {
                if (batch_ && !staged_.empty()) throw_on_error(vmhip_batch_run(batch_));
            }
            /// The same in two halves: the pass runs while the caller does something else (staging the next frames on
            /// a second engine, for one), and wait() blocks until it is done. fetch(), detect() and visible_counts()
            /// need the wait.
            void run_async() const {
                if (batch_ && !staged_.empty()) throw_on_error(vmhip_batch_run_async(batch_));
            }
            void wait() const {
                if (batch_ && !staged_.empty()) throw_on_error(vmhip_batch_wait(batch_));
            }
            /// Download the results of the last run.
            template <template <typename> class Model>
            std::vector<ClassifiedMesh<Scalar, Model<Scalar>::N_NEIGHBOURS>> fetch() const {
                constexpr int N = Model<Scalar>::N_NEIGHBOURS;
                const size_t n = staged_.size();
                std::vector<ClassifiedMesh<Scalar, N>> out(n);
                if (n == 0) return out;
                const int classes = vmhip_engine_n_classes(engine_);
                std::vector<int32_t> visible(n);
                throw_on_error(vmhip_batch_counts(batch_, visible.data()));
                std::vector<vmhip_result> results(n);
                for (size_t i = 0; i < n; ++i) {
                    const int V = visible[i];
                    vmhip_result& r = results[i];
                    std::memset(&r, 0, sizeof(r));
                    r.capacity = V;
                    if (V == 0) continue;
                    out[i].pixel_coordinates.resize(V);
                    out[i].global_indices.resize(V);
                    out[i].neighbourhood.resize(size_t(V) + 1);
                    out[i].classifications.resize((size_t(V) + 1) * classes);
                    r.pixel_coordinates = reinterpret_cast<float*>(out[i].pixel_coordinates.data());
                    r.global_indices = out[i].global_indices.data();
                    r.neighbourhood = reinterpret_cast<int32_t*>(out[i].neighbourhood.data());
                    r.classifications = out[i].classifications.data();
                }
                throw_on_error(vmhip_batch_fetch(batch_, results.data()));
                return out;
            }
            /// fetch() into arrays of the caller's (see vmhip_result; results[i].capacity rows each), one entry per
            /// staged frame. With arrays from vmhip_host_alloc the copies run at the full speed of the bus and nothing
            /// is copied a second time on the host: 1.6 ms instead of 14 ms for the 50 MB of a 16-frame batch.
            void fetch_into(std::vector<vmhip_result>& results) const {
                if (results.size() != staged_.size()) throw std::invalid_argument("fetch_into: one result per staged frame");
                if (!results.empty()) throw_on_error(vmhip_batch_fetch(batch_, results.data()));
            }
            /// fetch_into in two halves: the copies are queued and run while the caller does something else (with
            /// page-locked arrays; e.g. staging the next frames into another engine), fetch_wait() finishes them.
            void fetch_into_async(std::vector<vmhip_result>& results) const {
                if (results.size() != staged_.size()) throw std::invalid_argument("fetch_into_async: one result per staged frame");
                if (!results.empty()) throw_on_error(vmhip_batch_fetch_async(batch_, results.data()));
            }
            void fetch_wait() const {
                if (batch_ && !staged_.empty()) throw_on_error(vmhip_batch_fetch_wait(batch_));
            }
            /// fetch_into_async as one transfer: all frames' arrays are gathered on the device and come home in a single copy
            /// into `block` (page-locked, at least packed_size() bytes); results[i] point into it. Finished by fetch_wait().
            size_t packed_size() const { return batch_ ? vmhip_batch_fetch_packed_size(batch_) : 0; }
            void fetch_packed_async(void* block, size_t bytes, std::vector<vmhip_result>& results) const {
                results.assign(staged_.size(), vmhip_result{});
                if (!results.empty()) throw_on_error(vmhip_batch_fetch_packed_async(batch_, block, bytes, results.data()));
            }
            /// The nodes of one class among the results of the last run, picked and clustered on the device so that
            /// only they are downloaded (the reference's consumers walk the whole ClassifiedMesh on the host,
            /// example/draw.hpp:41-59).
            struct Detections {
                std::vector<int32_t> node;                    ///< index into the mesh, in the order of the visible nodes
                std::vector<std::array<Scalar, 2>> pixel;
                std::vector<Scalar> probability;
                std::vector<int32_t> cluster;                 ///< connected component (over the neighbourhood graph) of each
                std::vector<int32_t> cluster_size;
                std::vector<std::array<Scalar, 4>> cluster_box;     ///< min x, min y, max x, max y
                std::vector<std::array<Scalar, 2>> cluster_centre;  ///< mean pixel
            };
            /// A node is detected if its probability of `class_index` is at least `threshold` and, with `arg_max_only`,
            /// no other class has a larger one. One entry per staged frame.
            std::vector<Detections> detect(int class_index, Scalar threshold, bool arg_max_only = false, bool clusters = true) const {
                const size_t n = staged_.size();
                std::vector<Detections> out(n);
                if (n == 0) return out;
                std::vector<vmhip_detections> raw(n);
                for (auto& r : raw) std::memset(&r, 0, sizeof(r));
                /* first call sizes (capacity 0 fits only empty frames), second call copies */
                int rc = vmhip_batch_detect(batch_, class_index, float(threshold), arg_max_only, clusters, raw.data());
                if (rc == VMHIP_ERR_CAPACITY) {
                    for (size_t i = 0; i < n; ++i) {
                        Detections& d = out[i];
                        vmhip_detections& r = raw[i];
                        d.node.resize(r.n_detections);
                        d.pixel.resize(r.n_detections);
                        d.probability.resize(r.n_detections);
                        d.cluster.resize(clusters ? r.n_detections : 0);
                        d.cluster_size.resize(r.n_clusters);
                        d.cluster_box.resize(r.n_clusters);
                        d.cluster_centre.resize(r.n_clusters);
                        r.capacity = r.n_detections;
                        r.cluster_capacity = r.n_clusters;
                        r.node = d.node.data();
                        r.pixel = reinterpret_cast<float*>(d.pixel.data());
                        r.probability = d.probability.data();
                        r.cluster = clusters ? d.cluster.data() : nullptr;
                        r.cluster_size = d.cluster_size.data();
                        r.cluster_box = reinterpret_cast<float*>(d.cluster_box.data());
                        r.cluster_centre = reinterpret_cast<float*>(d.cluster_centre.data());
                    }
                    rc = vmhip_batch_detect(batch_, class_index, float(threshold), arg_max_only, clusters, raw.data());
                }
                throw_on_error(rc);
                return out;
            }
            /// What the training pipeline's LookupVisualMesh op returns (reference tensorflow/lookup.cpp:186-249), for
            /// every staged frame (no run needed): per node of the frame's lookup ranges its unit vector and a row
            /// [own position, positions of its neighbours along the ranges]. A neighbour outside the ranges is
            /// std::numeric_limits<int>::lowest() with HARD edges, the node's own position with SAME edges
            /// (training/dataset/projection/visual_mesh.py:82-89). Pixel coordinates (x, y) go along, on screen or not.
            enum EdgeType { HARD = VMHIP_EDGE_HARD, SAME = VMHIP_EDGE_SAME };
            template <int N>
            struct LookupGraph {
                std::vector<std::array<Scalar, 3>> vectors;
                std::vector<std::array<int32_t, N + 1>> graph;
                std::vector<std::array<Scalar, 2>> pixel_coordinates;
            };
            template <template <typename> class Model>
            std::vector<LookupGraph<Model<Scalar>::N_NEIGHBOURS>> lookup_graph(EdgeType edges = HARD) const {
                constexpr int N = Model<Scalar>::N_NEIGHBOURS;
                const size_t n = staged_.size();
                std::vector<LookupGraph<N>> out(n);
                if (n == 0) return out;
                std::vector<vmhip_lookup_export> raw(n);
                for (auto& r : raw) std::memset(&r, 0, sizeof(r));
                /* first call sizes (capacity 0 fits only empty frames), second call copies */
                int rc = vmhip_batch_export(batch_, int32_t(edges), raw.data());
                if (rc == VMHIP_ERR_CAPACITY) {
                    for (size_t i = 0; i < n; ++i) {
                        out[i].vectors.resize(raw[i].n_points);
                        out[i].graph.resize(raw[i].n_points);
                        out[i].pixel_coordinates.resize(raw[i].n_points);
                        raw[i].capacity = raw[i].n_points;
                        raw[i].vectors = reinterpret_cast<float*>(out[i].vectors.data());
                        raw[i].graph = reinterpret_cast<int32_t*>(out[i].graph.data());
                        raw[i].pixels = reinterpret_cast<float*>(out[i].pixel_coordinates.data());
                    }
                    rc = vmhip_batch_export(batch_, int32_t(edges), raw.data());
                }
                throw_on_error(rc);
                return out;
            }
            /// Visible nodes per staged frame after run().
            std::vector<int32_t> visible_counts() const {
                std::vector<int32_t> v(staged_.size());
                if (!v.empty()) throw_on_error(vmhip_batch_counts(batch_, v.data()));
                return v;
            }
            /// Where stage() looks up the nodes that may be on screen: on the host (Mesh::lookup, shared by a few
            /// threads; the default) or on the device, by a kernel that walks the same cone tree with the same
            /// comparisons. The single-frame calls always use the host (they size their results by the lookup).
            /// Needs a Mesh that exposes its cone tree (VISUALMESH_MESH_HAS_CONE_TREE); otherwise the host's lookup stays
#if defined(VISUALMESH_MESH_HAS_CONE_TREE)
            void set_device_lookup(bool on) { device_lookup_ = on; }
#else
            void set_device_lookup(bool) {}
#endif
            bool device_lookup() const { return device_lookup_; }
            /// The batch object behind stage/run/fetch, for profiling hooks.
            vmhip_batch* native_batch() const { return batch_; }
            /// How this engine's passes reached the stream so far: captured into a HIP graph, launched as a replay of a
            /// captured graph, launched kernel by kernel. A captured pass outlives the frames it was captured with
            /// (vmhip_batch_graph_stats), so an engine that is handed frame after frame of similar size captures once.
            struct GraphStats {
                int64_t captures = 0, graph_launches = 0, eager_launches = 0;
            };
            GraphStats graph_stats() const {
                GraphStats s;
                if (batch_) throw_on_error(vmhip_batch_graph_stats(batch_, &s.captures, &s.graph_launches, &s.eager_launches));
                return s;
            }
            /// Width of the classification rows (known once the engine has been used; -1 before).
            int n_classes() const { return engine_ ? int(vmhip_engine_n_classes(engine_)) : -1; }

            /// Forget the device copies of all meshes (same purpose as the reference OpenCL engine's
            /// clear_cache, engine/opencl/engine.hpp:559-572). Not needed for correctness: a cached copy is only
            /// reused for a mesh with the same address, node storage, node count and content fingerprint, so a
            /// different mesh that the allocator places where an old one lived is uploaded afresh (the reference
            /// OpenCL engine keys its cache on the address alone, engine/opencl/engine.hpp:603-625).
            void clear_cache() {
                for (auto& kv : meshes_) vmhip_mesh_release(kv.second.device);
                meshes_.clear();
                cache_bytes_ = 0;
                staged_.clear();  // a staged batch would point at released meshes
            }
            /// Device memory the mesh cache may hold before the least recently used meshes are released (meshes of
            /// the currently staged batch are never released). Default 8 GiB: a VisualMesh of many heights stays
            /// resident, an unbounded stream of distinct meshes does not grow without limit.
            void set_cache_limit(size_t bytes) { cache_limit_ = bytes; }
            size_t cache_bytes() const { return cache_bytes_; }
            size_t cached_meshes() const { return meshes_.size(); }

        private:
            struct FlatLayer {
                int32_t n_in, n_out, activation;
                std::vector<float> weights, biases;
            };
            struct MeshEntry {
                const void* nodes;
                size_t count;
                uint64_t fingerprint;
                vmhip_mesh* device;
                size_t bytes;
                uint64_t last_use;
                uint64_t pinned_by;  ///< the staging (staged_since_) that last used the mesh
            };
            struct FrameData {
                vmhip_frame frame;
                std::vector<int32_t> ranges;
                int32_t candidates = 0;
                bool lookup_on_device = false;  ///< the frame carries `lookup` instead of ranges
                vmhip_lookup lookup;
            };

            vmhip_engine* handle(int n_neighbours) const {
                if (engine_ && engine_nn_ == n_neighbours) return engine_;
                if (engine_) throw std::invalid_argument("this engine was already used with a different neighbour count");
                std::vector<vmhip_layer> flat(layers_.size());
                for (size_t i = 0; i < layers_.size(); ++i)
                    flat[i] = vmhip_layer{layers_[i].n_in, layers_[i].n_out, layers_[i].activation, layers_[i].weights.data(),
                                          layers_[i].biases.data()};
                vmhip_network net{int32_t(group_sizes_.size()), group_sizes_.data(), flat.data()};
                throw_on_error(vmhip_engine_create(&net, n_neighbours, int32_t(precision_), &engine_));
                engine_nn_ = n_neighbours;
                return engine_;
            }

            /// Over the limit: release least recently used meshes, but none that the staged batch or the running
            /// call (stamped `now`) uses.
            void trim_cache(uint64_t now) const {
                while (cache_bytes_ > cache_limit_) {
                    auto victim = meshes_.end();
                    for (auto e = meshes_.begin(); e != meshes_.end(); ++e) {
                        const bool staged = !staged_.empty() && e->second.pinned_by == staged_since_;
                        if (!staged && e->second.last_use < now && (victim == meshes_.end() || e->second.last_use < victim->second.last_use)) victim = e;
                    }
                    if (victim == meshes_.end()) break;
                    vmhip_mesh_release(victim->second.device);
                    cache_bytes_ -= victim->second.bytes;
                    meshes_.erase(victim);
                }
            }

            template <template <typename> class Model>
            vmhip_mesh* device_mesh(const Mesh<Scalar, Model>& mesh) const {
                constexpr int N = Model<Scalar>::N_NEIGHBOURS;
                const size_t n = mesh.nodes.size();
                /* FNV-1a over 64 evenly spaced nodes: tells meshes apart that share address, storage and size */
                uint64_t fingerprint = 1469598103934665603ull;
                for (size_t k = 0; k < 64 && n > 0; ++k) {
                    const unsigned char* bytes = reinterpret_cast<const unsigned char*>(&mesh.nodes[(k * (n - 1)) / 63]);
                    for (size_t b = 0; b < sizeof(mesh.nodes[0]); ++b) fingerprint = (fingerprint ^ bytes[b]) * 1099511628211ull;
                }
                auto it = meshes_.find(&mesh);
                if (it != meshes_.end() && it->second.nodes == mesh.nodes.data() && it->second.count == n && it->second.fingerprint == fingerprint) {
                    it->second.last_use = ++clock_;
                    if (staging_) it->second.pinned_by = staged_since_;
                    trim_cache(it->second.last_use);
                    return it->second.device;
                }
                if (it != meshes_.end()) {  // another mesh now lives at this address
                    vmhip_mesh_release(it->second.device);
                    cache_bytes_ -= it->second.bytes;
                    meshes_.erase(it);
                }
                std::vector<float> rays(n * 3);
                std::vector<int32_t> nbr(n * N);
                for (size_t i = 0; i < n; ++i) {
                    for (int c = 0; c < 3; ++c) rays[i * 3 + c] = mesh.nodes[i].ray[c];
                    for (int t = 0; t < N; ++t) nbr[i * N + t] = mesh.nodes[i].neighbours[t];
                }
                vmhip_mesh* dev = nullptr;
                throw_on_error(vmhip_mesh_upload(rays.data(), nbr.data(), int32_t(n), N, &dev));
#if defined(VISUALMESH_MESH_HAS_CONE_TREE)
                {  // the cone tree goes along, for lookups on the device
                    const auto& elements = mesh.tree().elements();
                    std::vector<vmhip_tree_element> tree(elements.size());
                    for (size_t i = 0; i < elements.size(); ++i) {
                        const auto& e = elements[i];
                        tree[i] = vmhip_tree_element{e.first, e.last, {e.child[0], e.child[1]}, {e.cone.axis[0], e.cone.axis[1], e.cone.axis[2]}, e.cone.c, e.cone.s};
                    }
                    const int rc = tree.empty() ? VMHIP_OK : vmhip_mesh_attach_tree(dev, tree.data(), int32_t(tree.size()));
                    if (rc != VMHIP_OK) {
                        vmhip_mesh_release(dev);
                        throw_on_error(rc);
                    }
                }
#endif
                const size_t bytes = n * (3 * sizeof(float) + N * sizeof(int32_t));
                const uint64_t now = ++clock_;
                meshes_[&mesh] = MeshEntry{mesh.nodes.data(), n, fingerprint, dev, bytes, now, staging_ ? staged_since_ : 0};
                cache_bytes_ += bytes;
                trim_cache(now);
                return dev;
            }

            /// The host side of the path: the mesh's lookup, flattened for the C ABI. Touches nothing but `fd`.
            template <template <typename> class Model>
            static void find_ranges(const Mesh<Scalar, Model>& mesh, const mat4<Scalar>& Hoc, const Lens<Scalar>& lens, FrameData& fd) {
                const auto ranges = mesh.lookup(Hoc, lens);
                fd.ranges.resize(ranges.size() * 2);
                fd.candidates = 0;
                for (size_t i = 0; i < ranges.size(); ++i) {
                    fd.ranges[2 * i] = ranges[i].first;
                    fd.ranges[2 * i + 1] = ranges[i].second;
                    fd.candidates += ranges[i].second - ranges[i].first;
                }
            }
            /// Everything else about a frame whose ranges are known.
            template <template <typename> class Model>
            void describe(const Mesh<Scalar, Model>& mesh, const mat4<Scalar>& Hoc, const Lens<Scalar>& lens, const void* image,
                          uint32_t format, FrameData& fd) const {
                vmhip_frame& f = fd.frame;
                std::memset(&f, 0, sizeof(f));
                f.mesh = device_mesh(mesh);
                for (int i = 0; i < 3; ++i)
                    for (int j = 0; j < 3; ++j) f.Rco[i * 3 + j] = Hoc[j][i];
                f.lens.width = lens.dimensions[0];
                f.lens.height = lens.dimensions[1];
                f.lens.projection = int32_t(lens.projection);
                f.lens.focal_length = lens.focal_length;
                f.lens.centre[0] = lens.centre[0];
                f.lens.centre[1] = lens.centre[1];
                f.lens.k[0] = lens.k[0];
                f.lens.k[1] = lens.k[1];
                f.lens.fov = lens.fov;
                f.ranges = fd.ranges.data();
                f.n_ranges = int32_t(fd.ranges.size() / 2);
#if defined(VISUALMESH_MESH_HAS_CONE_TREE)
                if (fd.lookup_on_device) {
                    const auto p = detail::ConeTree::lookup_parameters(Hoc, lens);
                    fd.lookup.cos_half_fov = p.cos_half_fov;
                    fd.lookup.sin_half_fov = p.sin_half_fov;
                    for (int i = 0; i < 4; ++i) {
                        for (int c = 0; c < 3; ++c) fd.lookup.edge[i][c] = p.edges[i].axis[c];
                        fd.lookup.edge[i][3] = p.edges[i].c;
                        fd.lookup.edge[i][4] = p.edges[i].s;
                    }
                    f.lookup = &fd.lookup;
                }
#endif
                f.image = image;
                f.fourcc = format;
            }

            void release() {
                if (batch_) vmhip_batch_destroy(batch_);
                batch_ = nullptr;
                clear_cache();
                if (engine_) vmhip_engine_destroy(engine_);
                engine_ = nullptr;
            }

            Precision precision_ = Precision::FP32;
            std::vector<int32_t> group_sizes_;
            std::vector<FlatLayer> layers_;
            mutable vmhip_engine* engine_ = nullptr;
            mutable int engine_nn_ = -1;
            mutable vmhip_batch* batch_ = nullptr;
            mutable std::map<const void*, MeshEntry> meshes_;
            mutable uint64_t clock_ = 0, staged_since_ = 0;
            mutable bool staging_ = false;
            bool device_lookup_ = false;
            mutable size_t cache_bytes_ = 0, cache_limit_ = size_t(8) << 30;
            mutable std::vector<FrameData> staged_;
        };

        /**
         * Scalar = double (the reference's engines are templates over Scalar, engine/cpu/engine.hpp:49-50): the reference
         * interface - construction from a NetworkStructure<double>, projection and classification of a
         * Mesh<double, Model> or VisualMesh<double, Model> - with every stage in fp64 on the device. It is the engine for
         * callers that need the reference's double results; the batch pipeline, the lookup on the device and the
         * detections of Engine<float> are not offered here. One frame per call.
         */
        template <>
        class Engine<double> {
            typedef double Scalar;

        public:
            template <template <typename> class Model>
            struct Frame {
                const Mesh<Scalar, Model>* mesh;
                mat4<Scalar> Hoc;
                Lens<Scalar> lens;
                const void* image;
                uint32_t format;
            };

            Engine(const NetworkStructure<Scalar>& structure = {}, Precision precision = Precision::FP64) {
                if (precision != Precision::FP64) throw std::invalid_argument("Engine<double> computes in fp64");
                for (const auto& group : structure) {
                    group_sizes_.push_back(int32_t(group.size()));
                    for (const auto& layer : group) {
                        FlatLayer flat;
                        flat.n_in = int32_t(layer.weights.size());
                        flat.n_out = int32_t(layer.biases.size());
                        flat.activation = int32_t(layer.activation);
                        flat.weights.reserve(size_t(flat.n_in) * flat.n_out);
                        for (const auto& row : layer.weights) {
                            if (int32_t(row.size()) != flat.n_out) throw std::invalid_argument("ragged weight matrix");
                            flat.weights.insert(flat.weights.end(), row.begin(), row.end());
                        }
                        flat.biases = layer.biases;
                        layers_.push_back(std::move(flat));
                    }
                }
            }
            ~Engine() { release(); }
            Engine(const Engine&) = delete;
            Engine& operator=(const Engine&) = delete;

            template <template <typename> class Model>
            ProjectedMesh<Scalar, Model<Scalar>::N_NEIGHBOURS> operator()(const Mesh<Scalar, Model>& mesh, const mat4<Scalar>& Hoc,
                                                                          const Lens<Scalar>& lens) const {
                constexpr int N = Model<Scalar>::N_NEIGHBOURS;
                ProjectedMesh<Scalar, N> out;
                std::array<int, N> null_row;
                null_row.fill(0);
                std::vector<int32_t> ranges;
                vmhip_frame_f64 f = describe(mesh, Hoc, lens, nullptr, 0, ranges);
                const int candidates = count(ranges);
                vmhip_result_f64 r{};
                if (candidates > 0) {
                    out.pixel_coordinates.resize(candidates);
                    out.global_indices.resize(candidates);
                    out.neighbourhood.resize(size_t(candidates) + 1);
                    r.capacity = candidates;
                    r.pixel_coordinates = reinterpret_cast<double*>(out.pixel_coordinates.data());
                    r.global_indices = out.global_indices.data();
                    r.neighbourhood = reinterpret_cast<int32_t*>(out.neighbourhood.data());
                    throw_on_error(vmhip_project_f64(handle(N), &f, &r));
                }
                /* nothing visible: the neighbourhood table is its null row alone, pointing at itself (reference
                 * engine/cpu/engine.hpp:127-143 with n_points = 0) */
                out.pixel_coordinates.resize(r.n_visible);
                out.global_indices.resize(r.n_visible);
                out.neighbourhood.resize(size_t(r.n_visible) + 1);
                if (r.n_visible == 0) out.neighbourhood[0] = null_row;
                return out;
            }
            template <template <typename> class Model>
            ProjectedMesh<Scalar, Model<Scalar>::N_NEIGHBOURS> operator()(const VisualMesh<Scalar, Model>& mesh, const mat4<Scalar>& Hoc,
                                                                          const Lens<Scalar>& lens) const {
                return operator()(mesh.height(Hoc[2][3]), Hoc, lens);
            }
            template <typename AnyMesh>
            auto project(const AnyMesh& mesh, const mat4<Scalar>& Hoc, const Lens<Scalar>& lens) const
              -> decltype(this->operator()(mesh, Hoc, lens)) {
                return operator()(mesh, Hoc, lens);
            }

            template <template <typename> class Model>
            ClassifiedMesh<Scalar, Model<Scalar>::N_NEIGHBOURS> operator()(const Mesh<Scalar, Model>& mesh, const mat4<Scalar>& Hoc,
                                                                           const Lens<Scalar>& lens, const void* image,
                                                                           const uint32_t& format) const {
                constexpr int N = Model<Scalar>::N_NEIGHBOURS;
                ClassifiedMesh<Scalar, N> out;
                std::vector<int32_t> ranges;
                vmhip_frame_f64 f = describe(mesh, Hoc, lens, image, format, ranges);
                const int candidates = count(ranges);
                vmhip_engine_f64* e = handle(N);
                const int classes = vmhip_engine_n_classes_f64(e);
                vmhip_result_f64 r{};
                out.pixel_coordinates.resize(candidates);
                out.global_indices.resize(candidates);
                out.neighbourhood.resize(size_t(candidates) + 1);
                out.classifications.resize((size_t(candidates) + 1) * classes);
                r.capacity = candidates;
                r.pixel_coordinates = reinterpret_cast<double*>(out.pixel_coordinates.data());
                r.global_indices = out.global_indices.data();
                r.neighbourhood = reinterpret_cast<int32_t*>(out.neighbourhood.data());
                r.classifications = out.classifications.data();
                /* called with no candidates too, so that an unsupported format throws as in the reference */
                throw_on_error(vmhip_classify_f64(e, &f, &r));
                if (r.n_visible == 0) return ClassifiedMesh<Scalar, N>();  // reference engine/cpu/engine.hpp:193
                out.pixel_coordinates.resize(r.n_visible);
                out.global_indices.resize(r.n_visible);
                out.neighbourhood.resize(size_t(r.n_visible) + 1);
                out.classifications.resize((size_t(r.n_visible) + 1) * classes);
                return out;
            }
            template <template <typename> class Model>
            ClassifiedMesh<Scalar, Model<Scalar>::N_NEIGHBOURS> operator()(const VisualMesh<Scalar, Model>& mesh, const mat4<Scalar>& Hoc,
                                                                           const Lens<Scalar>& lens, const void* image,
                                                                           const uint32_t& format) const {
                return operator()(mesh.height(Hoc[2][3]), Hoc, lens, image, format);
            }
            /// Independent frames, one after the other.
            template <template <typename> class Model>
            std::vector<ClassifiedMesh<Scalar, Model<Scalar>::N_NEIGHBOURS>> classify(const std::vector<Frame<Model>>& frames) const {
                std::vector<ClassifiedMesh<Scalar, Model<Scalar>::N_NEIGHBOURS>> out;
                out.reserve(frames.size());
                for (const auto& f : frames) out.push_back(operator()(*f.mesh, f.Hoc, f.lens, f.image, f.format));
                return out;
            }

            /// What the edge guard did since the engine was made: near-edge nodes the device listed and device decisions
            /// the host overruled.
            std::pair<int64_t, int64_t> guard_stats() const {
                int64_t listed = 0, overruled = 0;
                if (engine_) throw_on_error(vmhip_engine_guard_stats_f64(engine_, &listed, &overruled));
                return std::make_pair(listed, overruled);
            }
            void clear_cache() {
                for (auto& kv : meshes_) vmhip_mesh_release_f64(kv.second.device);
                meshes_.clear();
            }

        private:
            struct FlatLayer {
                int32_t n_in, n_out, activation;
                std::vector<double> weights, biases;
            };
            struct MeshEntry {
                const void* nodes;
                size_t count;
                uint64_t fingerprint;
                vmhip_mesh_f64* device;
            };

            static int count(const std::vector<int32_t>& ranges) {
                int n = 0;
                for (size_t i = 0; i + 1 < ranges.size(); i += 2) n += ranges[i + 1] - ranges[i];
                return n;
            }

            vmhip_engine_f64* handle(int n_neighbours) const {
                if (engine_ && engine_nn_ == n_neighbours) return engine_;
                if (engine_) throw std::invalid_argument("this engine was already used with a different neighbour count");
                std::vector<vmhip_layer_f64> flat(layers_.size());
                for (size_t i = 0; i < layers_.size(); ++i)
                    flat[i] = vmhip_layer_f64{layers_[i].n_in, layers_[i].n_out, layers_[i].activation, layers_[i].weights.data(),
                                              layers_[i].biases.data()};
                vmhip_network_f64 net{int32_t(group_sizes_.size()), group_sizes_.data(), flat.data()};
                throw_on_error(vmhip_engine_create_f64(&net, n_neighbours, &engine_));
                engine_nn_ = n_neighbours;
                return engine_;
            }

            /// The device copy of a mesh, keyed like Engine<float>'s cache: address, node storage, node count and a
            /// fingerprint of the content.
            template <template <typename> class Model>
            vmhip_mesh_f64* device_mesh(const Mesh<Scalar, Model>& mesh) const {
                constexpr int N = Model<Scalar>::N_NEIGHBOURS;
                const size_t n = mesh.nodes.size();
                uint64_t fingerprint = 1469598103934665603ull;
                for (size_t k = 0; k < 64 && n > 0; ++k) {
                    const unsigned char* bytes = reinterpret_cast<const unsigned char*>(&mesh.nodes[(k * (n - 1)) / 63]);
                    for (size_t b = 0; b < sizeof(mesh.nodes[0]); ++b) fingerprint = (fingerprint ^ bytes[b]) * 1099511628211ull;
                }
                auto it = meshes_.find(&mesh);
                if (it != meshes_.end() && it->second.nodes == mesh.nodes.data() && it->second.count == n && it->second.fingerprint == fingerprint)
                    return it->second.device;
                if (it != meshes_.end()) {
                    vmhip_mesh_release_f64(it->second.device);
                    meshes_.erase(it);
                }
                std::vector<double> rays(n * 3);
                std::vector<int32_t> nbr(n * N);
                for (size_t i = 0; i < n; ++i) {
                    for (int c = 0; c < 3; ++c) rays[i * 3 + c] = mesh.nodes[i].ray[c];
                    for (int t = 0; t < N; ++t) nbr[i * N + t] = mesh.nodes[i].neighbours[t];
                }
                vmhip_mesh_f64* dev = nullptr;
                throw_on_error(vmhip_mesh_upload_f64(rays.data(), nbr.data(), int32_t(n), N, &dev));
                meshes_[&mesh] = MeshEntry{mesh.nodes.data(), n, fingerprint, dev};
                return dev;
            }

            template <template <typename> class Model>
            vmhip_frame_f64 describe(const Mesh<Scalar, Model>& mesh, const mat4<Scalar>& Hoc, const Lens<Scalar>& lens, const void* image,
                                     uint32_t format, std::vector<int32_t>& ranges) const {
                const auto found = mesh.lookup(Hoc, lens);
                ranges.resize(found.size() * 2);
                for (size_t i = 0; i < found.size(); ++i) ranges[2 * i] = found[i].first, ranges[2 * i + 1] = found[i].second;
                vmhip_frame_f64 f;
                std::memset(&f, 0, sizeof(f));
                f.mesh = device_mesh(mesh);
                for (int i = 0; i < 3; ++i)
                    for (int j = 0; j < 3; ++j) f.Rco[i * 3 + j] = Hoc[j][i];
                f.lens.width = lens.dimensions[0];
                f.lens.height = lens.dimensions[1];
                f.lens.projection = int32_t(lens.projection);
                f.lens.focal_length = lens.focal_length;
                f.lens.centre[0] = lens.centre[0], f.lens.centre[1] = lens.centre[1];
                f.lens.k[0] = lens.k[0], f.lens.k[1] = lens.k[1];
                f.lens.fov = lens.fov;
                f.ranges = ranges.data();
                f.n_ranges = int32_t(found.size());
                f.image = image;
                f.fourcc = format;
                return f;
            }

            void release() {
                clear_cache();
                if (engine_) vmhip_engine_destroy_f64(engine_);
                engine_ = nullptr;
            }

            std::vector<int32_t> group_sizes_;
            std::vector<FlatLayer> layers_;
            mutable vmhip_engine_f64* engine_ = nullptr;
            mutable int engine_nn_ = -1;
            mutable std::map<const void*, MeshEntry> meshes_;
        };

        /**
         * Three engines taking turns, so that the upload of one batch, the kernels of the one before and the download of
         * the one before that run at the same time: what a caller otherwise writes by hand with stage_async / run_async /
         * wait / fetch_into_async / fetch_wait on three Engine objects. No counterpart in the reference, whose benchmark
         * runs one frame at a time per engine (example/benchmark.cpp:50-58).
         *
         *     Pipeline<float> pipe(network);
         *     for (;;) { if (auto* done = pipe.submit(next_frames())) consume(*done); }   // results of the batch two submits ago
         *     while (auto* done = pipe.flush()) consume(*done);
         *
         * The frames' images must lie in page-locked memory (vmhip_host_alloc; a batch's images in one allocation go up as one
         * copy) and stay untouched until the next submit() or flush() has returned. The results returned point into page-locked
         * memory of the pipeline and stay valid until two more calls of submit() or flush().
         */
        template <typename Scalar>
        class Pipeline {
            static_assert(std::is_same<Scalar, float>::value, "the pipeline drives Engine<float>");

        public:
            explicit Pipeline(const NetworkStructure<Scalar>& structure = {}, Precision precision = Precision::FP32) {
                for (Slot& s : slots_) s.engine.reset(new Engine<Scalar>(structure, precision));
            }
            ~Pipeline() {
                for (Slot& s : slots_) {
                    try {
                        if (s.running) s.engine->wait();
                        if (s.fetching) s.engine->fetch_wait();
                    } catch (...) {
                    }
                    if (s.block) vmhip_host_free(s.block);
                }
            }
            Pipeline(const Pipeline&) = delete;
            Pipeline& operator=(const Pipeline&) = delete;

            /// Queue a batch; returns the results of the batch submitted two calls earlier (one entry per frame of that batch:
            /// n_visible and pointers as in vmhip_result), or nullptr while the pipeline fills.
            template <template <typename> class Model>
            const std::vector<vmhip_result>* submit(const std::vector<typename Engine<Scalar>::template Frame<Model>>& frames) {
                Slot& now = slots_[step_ % 3];
                now.engine->stage_async(frames);
                now.engine->run_async();
                now.running = true;
                now.neighbours = Model<Scalar>::N_NEIGHBOURS;
                return advance();
            }
            /// Drain: the results of the batches still in flight, oldest first, then nullptr.
            const std::vector<vmhip_result>* flush() {
                for (int turn = 0; turn < 2; ++turn) {
                    bool in_flight = false;
                    for (const Slot& s : slots_) in_flight = in_flight || s.running || s.fetching;
                    if (!in_flight) return nullptr;
                    if (const std::vector<vmhip_result>* done = advance()) return done;
                }
                return nullptr;
            }
            /// The engines, e.g. to set a cache limit or the lookup on the device on all three.
            Engine<Scalar>& engine(int i) { return *slots_[i % 3].engine; }
            /// Captures and launches of the three engines together (Engine::graph_stats).
            typename Engine<Scalar>::GraphStats graph_stats() const {
                typename Engine<Scalar>::GraphStats total;
                for (const Slot& s : slots_) {
                    const typename Engine<Scalar>::GraphStats one = s.engine->graph_stats();
                    total.captures += one.captures, total.graph_launches += one.graph_launches, total.eager_launches += one.eager_launches;
                }
                return total;
            }

        private:
            struct Slot {
                std::unique_ptr<Engine<Scalar>> engine;
                bool running = false, fetching = false;
                int neighbours = 0;
                void* block = nullptr;
                size_t block_bytes = 0;
                std::vector<vmhip_result> results;
            };
            static size_t pad(size_t n) { return (n + 255) / 256 * 256; }

            const std::vector<vmhip_result>* advance() {
                Slot& previous = slots_[(step_ + 2) % 3];  // submitted one call ago: its kernels finish, its download starts
                Slot& oldest = slots_[(step_ + 1) % 3];    // submitted two calls ago: its download finishes
                ++step_;
                /* The oldest batch's download is finished before the next one is queued: with the tail of one download and
                 * the head of the next in flight together, the upload that runs beside them takes longer (2.0-2.1 ms per
                 * batch instead of 1.8 on the benchmark's batches). */
                const std::vector<vmhip_result>* done = nullptr;
                if (previous.running) previous.engine->wait();
                if (oldest.fetching) {
                    oldest.engine->fetch_wait();
                    oldest.fetching = false;
                    done = &oldest.results;
                }
                if (previous.running) {
                    previous.running = false;
                    const std::vector<int32_t> visible = previous.engine->visible_counts();
                    const size_t classes = size_t(previous.engine->n_classes()), nn = size_t(previous.neighbours);
                    size_t need = 0;
                    for (int32_t v : visible)
                        if (v > 0) need += pad(8 * size_t(v)) + pad(4 * size_t(v)) + pad(4 * (size_t(v) + 1) * nn) + pad(4 * (size_t(v) + 1) * classes);
                    if (need > previous.block_bytes) {
                        if (previous.block) vmhip_host_free(previous.block);
                        previous.block = vmhip_host_alloc(need + need / 8);
                        previous.block_bytes = previous.block ? need + need / 8 : 0;
                        if (!previous.block) throw std::system_error(VMHIP_ERR_HIP, hip_error_category(), "Pipeline: no page-locked memory for the results");
                    }
                    previous.results.assign(visible.size(), vmhip_result{});
                    char* at = static_cast<char*>(previous.block);
                    for (size_t i = 0; i < visible.size(); ++i) {
                        const size_t v = size_t(visible[i]);
                        vmhip_result& r = previous.results[i];
                        r.capacity = int32_t(v);
                        if (v == 0) continue;
                        r.pixel_coordinates = reinterpret_cast<float*>(at), at += pad(8 * v);
                        r.global_indices = reinterpret_cast<int32_t*>(at), at += pad(4 * v);
                        r.neighbourhood = reinterpret_cast<int32_t*>(at), at += pad(4 * (v + 1) * nn);
                        r.classifications = reinterpret_cast<float*>(at), at += pad(4 * (v + 1) * classes);
                    }
                    previous.engine->fetch_into_async(previous.results);
                    previous.fetching = true;
                }
                return done;
            }

            std::array<Slot, 3> slots_;
            size_t step_ = 0;
        };

    }  // namespace hip
}  // namespace engine
}  // namespace visualmesh

#endif  // !defined(VISUALMESH_DISABLE_HIP)
#endif  // VISUALMESH_ENGINE_HIP_ENGINE_HPP

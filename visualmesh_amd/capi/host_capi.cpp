/*
 * host_capi.cpp - a small C interface over the C++ host code (Mesh, VisualMesh and
 * visualmesh::engine::hip::Engine), so that Python tests and the benchmark drive exactly the C++ a user
 * of the engine would write. Built into libvisualmesh_host.so, which links libvisualmesh_hip.so.
 *
 * Functions return a count / 0 on success or a negative status (the VMHIP_ERR_* values);
 * vmh_last_error() holds the message of the last failure on the calling thread.
 *
 * Compiled twice: as it stands for Scalar = float (libvisualmesh_host.so), and with -DVMH_DOUBLE for Scalar = double
 * (libvisualmesh_host_f64.so: the same names with `real` = double and the _f64 structures of visualmesh_hip.h; the
 * parts of Engine<float> that Engine<double> does not offer - staged batches, lookup graphs, model files - are left out).
 */
#include <chrono>
#include <cstring>
#include <memory>
#include <stdexcept>
#include <string>
#include <system_error>
#include <vector>

#include "visualmesh/engine/hip/engine.hpp"
#include "visualmesh/geometry/Circle.hpp"
#include "visualmesh/geometry/Sphere.hpp"
#include "visualmesh/mesh.hpp"
#include "visualmesh/model/nmgrid8.hpp"
#include "visualmesh/model/ring6.hpp"
#include "visualmesh/utility/load_model.hpp"
#include "visualmesh/visualmesh.hpp"

#if defined(VMH_DOUBLE)
typedef double real;
typedef vmhip_lens_f64 vmh_lens_t;
typedef vmhip_layer_f64 vmh_layer_t;
typedef vmhip_network_f64 vmh_network_t;
#else
typedef float real;
typedef vmhip_lens vmh_lens_t;
typedef vmhip_layer vmh_layer_t;
typedef vmhip_network vmh_network_t;
#endif

using namespace visualmesh;
using geometry::Circle;
using geometry::Sphere;
using model::NMGrid8;
using model::Ring6;
typedef engine::hip::Engine<real> HipEngine;

enum { VMH_RING6 = 0, VMH_NMGRID8 = 1 };
enum { VMH_SPHERE = 0, VMH_CIRCLE = 1 };

struct vmh_mesh {
    const Mesh<real, Ring6>* r6 = nullptr;
    const Mesh<real, NMGrid8>* g8 = nullptr;
    std::unique_ptr<Mesh<real, Ring6>> own_r6;
    std::unique_ptr<Mesh<real, NMGrid8>> own_g8;
};
struct vmh_visualmesh {
    std::unique_ptr<VisualMesh<real, Ring6>> r6;
    std::unique_ptr<VisualMesh<real, NMGrid8>> g8;
    std::vector<std::unique_ptr<vmh_mesh>> views;  // ascending height
};
#if !defined(VMH_DOUBLE)
struct vmh_model {
    ModelFile<real> file;
};
#endif
struct vmh_engine {
    int model;
    std::unique_ptr<HipEngine> engine;
    std::vector<ClassifiedMesh<real, 6>> fetched6;
    std::vector<ClassifiedMesh<real, 8>> fetched8;
};

namespace {
thread_local std::string g_error;

int report(const std::exception& e) {
    g_error = e.what();
    if (const std::system_error* se = dynamic_cast<const std::system_error*>(&e)) return se->code().value();
    if (g_error.find("Unsupported image format") != std::string::npos) return VMHIP_ERR_FORMAT;
    if (g_error.find("lens") != std::string::npos) return VMHIP_ERR_LENS;
    return VMHIP_ERR_ARGUMENT;
}
#define GUARD(...)                      \
    try {                               \
        __VA_ARGS__                     \
    } catch (const std::exception& e) { \
        return report(e);               \
    }

Lens<real> to_lens(const vmh_lens_t* l) {
    Lens<real> lens;
    lens.dimensions = {{l->width, l->height}};
    lens.projection = LensProjection(l->projection);
    lens.focal_length = l->focal_length;
    lens.centre = {{l->centre[0], l->centre[1]}};
    lens.k = {{l->k[0], l->k[1]}};
    lens.fov = l->fov;
    return lens;
}
mat4<real> to_hoc(const real* H) {
    mat4<real> m;
    for (int i = 0; i < 4; ++i)
        for (int j = 0; j < 4; ++j) m[i][j] = H[i * 4 + j];
    return m;
}
NetworkStructure<real> to_network(const vmh_network_t* net) {
    NetworkStructure<real> s;
    int li = 0;
    for (int g = 0; net && g < net->n_groups; ++g) {
        s.emplace_back();
        for (int l = 0; l < net->group_sizes[g]; ++l, ++li) {
            const vmh_layer_t& L = net->layers[li];
            Layer<real> layer;
            layer.weights.assign(L.n_in, std::vector<real>(L.n_out));
            for (int t = 0; t < L.n_in; ++t)
                for (int j = 0; j < L.n_out; ++j) layer.weights[t][j] = L.weights[size_t(t) * L.n_out + j];
            layer.biases.assign(L.biases, L.biases + L.n_out);
            layer.activation = ActivationFunction(L.activation);
            s.back().push_back(std::move(layer));
        }
    }
    return s;
}

template <typename M>
void copy_nodes(const M& mesh, real* rays, int32_t* nbr) {
    const int nn = M::N_NEIGHBOURS;
    for (size_t i = 0; i < mesh.nodes.size(); ++i) {
        if (rays)
            for (int c = 0; c < 3; ++c) rays[i * 3 + c] = mesh.nodes[i].ray[c];
        if (nbr)
            for (int t = 0; t < nn; ++t) nbr[i * nn + t] = mesh.nodes[i].neighbours[t];
    }
}

template <typename R>
int export_result(const R& r, int cap, real* px, int32_t* nb, int32_t* gidx) {
    const int V = int(r.global_indices.size());
    if (V > cap) {
        g_error = "result capacity too small";
        return VMHIP_ERR_CAPACITY;
    }
    /* an empty projection still has its null row (the caller's table holds cap + 1 rows); an empty classification has none */
    if (nb && !r.neighbourhood.empty()) std::memcpy(nb, r.neighbourhood.data(), sizeof(r.neighbourhood[0]) * r.neighbourhood.size());
    if (V == 0) return 0;
    if (px) std::memcpy(px, r.pixel_coordinates.data(), sizeof(real) * 2 * V);
    if (gidx) std::memcpy(gidx, r.global_indices.data(), sizeof(int32_t) * V);
    return V;
}
}  // namespace

extern "C" {

const char* vmh_last_error(void) { return g_error.c_str(); }

vmh_mesh* vmh_mesh_create(int model, int shape, real radius, real h, real k, real max_distance) {
    try {
        std::unique_ptr<vmh_mesh> m(new vmh_mesh());
        if (model == VMH_RING6) {
            if (shape == VMH_SPHERE) m->own_r6.reset(new Mesh<real, Ring6>(Sphere<real>(radius), h, k, max_distance));
            else if (shape == VMH_CIRCLE) m->own_r6.reset(new Mesh<real, Ring6>(Circle<real>(radius), h, k, max_distance));
            else return nullptr;
            m->r6 = m->own_r6.get();
        }
        else if (model == VMH_NMGRID8) {
            if (shape == VMH_SPHERE) m->own_g8.reset(new Mesh<real, NMGrid8>(Sphere<real>(radius), h, k, max_distance));
            else if (shape == VMH_CIRCLE) m->own_g8.reset(new Mesh<real, NMGrid8>(Circle<real>(radius), h, k, max_distance));
            else return nullptr;
            m->g8 = m->own_g8.get();
        }
        else return nullptr;
        return m.release();
    } catch (const std::exception& e) {
        g_error = e.what();
        return nullptr;
    }
}
void vmh_mesh_destroy(vmh_mesh* m) { delete m; }
int vmh_mesh_n_nodes(const vmh_mesh* m) { return m->r6 ? int(m->r6->nodes.size()) : int(m->g8->nodes.size()); }
int vmh_mesh_n_neighbours(const vmh_mesh* m) { return m->r6 ? 6 : 8; }
real vmh_mesh_h(const vmh_mesh* m) { return m->r6 ? m->r6->h : m->g8->h; }
void vmh_mesh_copy(const vmh_mesh* m, real* rays, int32_t* neighbours) {
    if (m->r6) copy_nodes(*m->r6, rays, neighbours);
    else copy_nodes(*m->g8, rays, neighbours);
}
int vmh_mesh_lookup(const vmh_mesh* m, const real* Hoc16, const vmh_lens_t* lens, int32_t* ranges, int cap) {
    GUARD({
        const auto r = m->r6 ? m->r6->lookup(to_hoc(Hoc16), to_lens(lens)) : m->g8->lookup(to_hoc(Hoc16), to_lens(lens));
        for (int i = 0; i < int(r.size()) && i < cap; ++i) {
            ranges[2 * i] = r[i].first;
            ranges[2 * i + 1] = r[i].second;
        }
        return int(r.size());
    })
}

vmh_visualmesh* vmh_visualmesh_create(int model, int shape, real radius, real min_h, real max_h, real k, real max_error,
                                      real max_distance) {
    try {
        std::unique_ptr<vmh_visualmesh> v(new vmh_visualmesh());
        if (model == VMH_RING6) {
            if (shape == VMH_SPHERE) v->r6.reset(new VisualMesh<real, Ring6>(Sphere<real>(radius), min_h, max_h, k, max_error, max_distance));
            else v->r6.reset(new VisualMesh<real, Ring6>(Circle<real>(radius), min_h, max_h, k, max_error, max_distance));
            for (const auto& kv : v->r6->meshes()) {
                std::unique_ptr<vmh_mesh> view(new vmh_mesh());
                view->r6 = &kv.second;
                v->views.push_back(std::move(view));
            }
        }
        else if (model == VMH_NMGRID8) {
            if (shape == VMH_SPHERE) v->g8.reset(new VisualMesh<real, NMGrid8>(Sphere<real>(radius), min_h, max_h, k, max_error, max_distance));
            else v->g8.reset(new VisualMesh<real, NMGrid8>(Circle<real>(radius), min_h, max_h, k, max_error, max_distance));
            for (const auto& kv : v->g8->meshes()) {
                std::unique_ptr<vmh_mesh> view(new vmh_mesh());
                view->g8 = &kv.second;
                v->views.push_back(std::move(view));
            }
        }
        else return nullptr;
        return v.release();
    } catch (const std::exception& e) {
        g_error = e.what();
        return nullptr;
    }
}
void vmh_visualmesh_destroy(vmh_visualmesh* v) { delete v; }
int vmh_visualmesh_n_meshes(const vmh_visualmesh* v) { return int(v->views.size()); }
const vmh_mesh* vmh_visualmesh_mesh(const vmh_visualmesh* v, int i) { return v->views[i].get(); }
const vmh_mesh* vmh_visualmesh_height(const vmh_visualmesh* v, real h) {
    const void* picked = v->r6 ? static_cast<const void*>(&v->r6->height(h)) : static_cast<const void*>(&v->g8->height(h));
    for (const auto& view : v->views)
        if (static_cast<const void*>(view->r6) == picked || static_cast<const void*>(view->g8) == picked) return view.get();
    return nullptr;
}

int vmh_engine_create(const vmh_network_t* net, int model, int precision, vmh_engine** out) {
    GUARD({
        std::unique_ptr<vmh_engine> e(new vmh_engine());
        e->model = model;
        e->engine.reset(new HipEngine(to_network(net), engine::hip::Precision(precision)));
        *out = e.release();
        return 0;
    })
}
void vmh_engine_destroy(vmh_engine* e) { delete e; }

int vmh_engine_project(vmh_engine* e, const vmh_mesh* m, const real* Hoc16, const vmh_lens_t* lens, int cap, real* px,
                       int32_t* nb, int32_t* gidx) {
    GUARD({
        if (m->r6) return export_result(e->engine->project(*m->r6, to_hoc(Hoc16), to_lens(lens)), cap, px, nb, gidx);
        return export_result(e->engine->project(*m->g8, to_hoc(Hoc16), to_lens(lens)), cap, px, nb, gidx);
    })
}

int vmh_engine_classify(vmh_engine* e, const vmh_mesh* m, const real* Hoc16, const vmh_lens_t* lens, const void* image,
                        uint32_t fourcc, int cap, real* px, int32_t* nb, int32_t* gidx, real* cls) {
    GUARD({
        if (m->r6) {
            const auto r = (*e->engine)(*m->r6, to_hoc(Hoc16), to_lens(lens), image, fourcc);
            const int V = export_result(r, cap, px, nb, gidx);
            if (V > 0 && cls) std::memcpy(cls, r.classifications.data(), sizeof(real) * r.classifications.size());
            return V;
        }
        const auto r = (*e->engine)(*m->g8, to_hoc(Hoc16), to_lens(lens), image, fourcc);
        const int V = export_result(r, cap, px, nb, gidx);
        if (V > 0 && cls) std::memcpy(cls, r.classifications.data(), sizeof(real) * r.classifications.size());
        return V;
    })
}

/* Average wall-clock milliseconds of `repeats` calls of engine(mesh, Hoc, lens, image, fourcc), results returned by value
 * and dropped: what one call of the reference's interface costs a C++ caller (reference example/benchmark.cpp:50-58
 * times exactly this). One untimed call comes first. */
int vmh_engine_time_calls(vmh_engine* e, const vmh_mesh* m, const real* Hoc16, const vmh_lens_t* lens, const void* image,
                          uint32_t fourcc, int repeats, double* ms_per_call) {
    GUARD({
        size_t visible = 0;
        const auto Hoc = to_hoc(Hoc16);
        const auto L = to_lens(lens);
        std::chrono::steady_clock::time_point t0;
        for (int i = -1; i < repeats; ++i) {
            if (i == 0) t0 = std::chrono::steady_clock::now();
            if (m->r6) visible += (*e->engine)(*m->r6, Hoc, L, image, fourcc).global_indices.size();
            else visible += (*e->engine)(*m->g8, Hoc, L, image, fourcc).global_indices.size();
        }
        *ms_per_call = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count() / (repeats > 0 ? repeats : 1);
        return int(visible / size_t(repeats + 1));
    })
}

#if defined(VMH_DOUBLE)
int vmh_engine_guard_stats(vmh_engine* e, int64_t* listed, int64_t* overruled) {
    GUARD({
        const auto stats = e->engine->guard_stats();
        *listed = stats.first, *overruled = stats.second;
        return 0;
    })
}
#else
/* staged batch: all frames must use meshes of the engine's model; wait = 0 queues the copies and returns (stage_async) */
int vmh_engine_stage(vmh_engine* e, int n, const vmh_mesh* const* meshes, const real* Hoc16s, const vmh_lens_t* lenses,
                     const void* const* images, const uint32_t* fourccs, int wait) {
    GUARD({
        if (e->model == VMH_RING6) {
            std::vector<HipEngine::Frame<Ring6>> frames(n);
            for (int i = 0; i < n; ++i) {
                if (!meshes[i]->r6) throw std::invalid_argument("mesh model does not match the engine");
                frames[i] = HipEngine::Frame<Ring6>{meshes[i]->r6, to_hoc(Hoc16s + 16 * i), to_lens(lenses + i), images[i], fourccs[i]};
            }
            if (wait) e->engine->stage(frames);
            else e->engine->stage_async(frames);
        }
        else {
            std::vector<HipEngine::Frame<NMGrid8>> frames(n);
            for (int i = 0; i < n; ++i) {
                if (!meshes[i]->g8) throw std::invalid_argument("mesh model does not match the engine");
                frames[i] = HipEngine::Frame<NMGrid8>{meshes[i]->g8, to_hoc(Hoc16s + 16 * i), to_lens(lenses + i), images[i], fourccs[i]};
            }
            if (wait) e->engine->stage(frames);
            else e->engine->stage_async(frames);
        }
        return 0;
    })
}
int vmh_engine_run(vmh_engine* e) {
    GUARD({
        e->engine->run();
        return 0;
    })
}
int vmh_engine_counts(vmh_engine* e, int32_t* visible, int n) {
    GUARD({
        const std::vector<int32_t> v = e->engine->visible_counts();
        for (int i = 0; i < n && i < int(v.size()); ++i) visible[i] = v[i];
        return int(v.size());
    })
}
/* downloads every frame of the last run into the harness */
int vmh_engine_fetch(vmh_engine* e) {
    GUARD({
        if (e->model == VMH_RING6) {
            e->fetched6 = e->engine->fetch<Ring6>();
            return int(e->fetched6.size());
        }
        e->fetched8 = e->engine->fetch<NMGrid8>();
        return int(e->fetched8.size());
    })
}
/* copies frame i of the last fetch */
int vmh_engine_result(vmh_engine* e, int i, int cap, real* px, int32_t* nb, int32_t* gidx, real* cls) {
    GUARD({
        if (e->model == VMH_RING6) {
            const auto& r = e->fetched6.at(i);
            const int V = export_result(r, cap, px, nb, gidx);
            if (V > 0 && cls) std::memcpy(cls, r.classifications.data(), sizeof(real) * r.classifications.size());
            return V;
        }
        const auto& r = e->fetched8.at(i);
        const int V = export_result(r, cap, px, nb, gidx);
        if (V > 0 && cls) std::memcpy(cls, r.classifications.data(), sizeof(real) * r.classifications.size());
        return V;
    })
}
/* lookup_graph() of staged frame i: returns its number of points; copies when the arrays hold that many rows */
int vmh_engine_lookup_graph(vmh_engine* e, int i, int same_edges, int cap, real* vectors, int32_t* graph, real* pixels) {
    GUARD({
        typedef HipEngine E;
        const E::EdgeType edges = same_edges ? E::SAME : E::HARD;
        if (e->model == VMH_RING6) {
            const auto all = e->engine->lookup_graph<Ring6>(edges);
            const auto& g = all.at(i);
            const int n = int(g.vectors.size());
            if (n <= cap && n > 0) {
                std::memcpy(vectors, g.vectors.data(), sizeof(real) * 3 * n);
                std::memcpy(graph, g.graph.data(), sizeof(int32_t) * 7 * n);
                if (pixels) std::memcpy(pixels, g.pixel_coordinates.data(), sizeof(real) * 2 * n);
            }
            return n;
        }
        const auto all = e->engine->lookup_graph<NMGrid8>(edges);
        const auto& g = all.at(i);
        const int n = int(g.vectors.size());
        if (n <= cap && n > 0) {
            std::memcpy(vectors, g.vectors.data(), sizeof(real) * 3 * n);
            std::memcpy(graph, g.graph.data(), sizeof(int32_t) * 9 * n);
            if (pixels) std::memcpy(pixels, g.pixel_coordinates.data(), sizeof(real) * 2 * n);
        }
        return n;
    })
}
void* vmh_engine_native_batch(vmh_engine* e) { return e->engine->native_batch(); }
void vmh_engine_clear_cache(vmh_engine* e) { e->engine->clear_cache(); }
void vmh_engine_set_device_lookup(vmh_engine* e, int on) {
    if (e && e->engine) e->engine->set_device_lookup(on != 0);
}
void vmh_engine_set_cache_limit(vmh_engine* e, uint64_t bytes) { e->engine->set_cache_limit(size_t(bytes)); }
int vmh_engine_cache_info(vmh_engine* e, uint64_t* bytes) {
    *bytes = e->engine->cache_bytes();
    return int(e->engine->cached_meshes());
}

/* ---- exported networks and dataset lens files (visualmesh/utility/load_model.hpp) ---- */
vmh_model* vmh_model_load(const char* path) {
    try {
        std::unique_ptr<vmh_model> m(new vmh_model());
        m->file = load_model_file<real>(path);
        return m.release();
    } catch (const std::exception& e) {
        report(e);
        return nullptr;
    }
}
void vmh_model_free(vmh_model* m) { delete m; }
/* names are copied into caller buffers of `cap` bytes */
int vmh_model_info(const vmh_model* m, char* mesh, char* shape, int cap, real* radius, real* intersections) {
    GUARD({
        if (cap <= 0) throw std::invalid_argument("model_info: no room for the names");
        std::strncpy(mesh, m->file.mesh.c_str(), size_t(cap) - 1);
        std::strncpy(shape, m->file.shape.c_str(), size_t(cap) - 1);
        mesh[cap - 1] = shape[cap - 1] = 0;
        *radius = m->file.radius;
        *intersections = m->file.intersections;
        return int(m->file.network.size());
    })
}
int vmh_model_group_size(const vmh_model* m, int group) {
    GUARD({ return int(m->file.network.at(group).size()); })
}
/* sizes of a layer; weights (row major [n_in][n_out]) and biases are copied when the pointers are not null */
int vmh_model_layer(const vmh_model* m, int group, int layer, int* n_in, int* n_out, int* activation, real* weights, real* biases) {
    GUARD({
        const Layer<real>& l = m->file.network.at(group).at(layer);
        *n_in = int(l.weights.size());
        *n_out = int(l.biases.size());
        *activation = int(l.activation);
        if (weights)
            for (size_t r = 0; r < l.weights.size(); ++r) std::memcpy(weights + r * l.biases.size(), l.weights[r].data(), sizeof(real) * l.biases.size());
        if (biases) std::memcpy(biases, l.biases.data(), sizeof(real) * l.biases.size());
        return 0;
    })
}
int vmh_lens_load(const char* path, int width, int height, vmh_lens_t* lens, real* Hoc16) {
    GUARD({
        const LensFile<real> f = load_lens<real>(path, width, height);
        lens->width = width;
        lens->height = height;
        lens->projection = int(f.lens.projection);
        lens->focal_length = f.lens.focal_length;
        lens->centre[0] = f.lens.centre[0], lens->centre[1] = f.lens.centre[1];
        lens->k[0] = f.lens.k[0], lens->k[1] = f.lens.k[1];
        lens->fov = f.lens.fov;
        for (int r = 0; r < 4; ++r)
            for (int c = 0; c < 4; ++c) Hoc16[r * 4 + c] = f.Hoc[r][c];
        return 0;
    })
}

/* ---- Pipeline<float>: three engines in rotation ---- */
struct vmh_pipeline {
    int model;
    std::unique_ptr<engine::hip::Pipeline<real>> pipe;
    const std::vector<vmhip_result>* done = nullptr;
};
int vmh_pipeline_create(const vmh_network_t* net, int model, int precision, vmh_pipeline** out) {
    GUARD({
        std::unique_ptr<vmh_pipeline> p(new vmh_pipeline());
        p->model = model;
        p->pipe.reset(new engine::hip::Pipeline<real>(to_network(net), engine::hip::Precision(precision)));
        *out = p.release();
        return 0;
    })
}
void vmh_pipeline_destroy(vmh_pipeline* p) { delete p; }
/* queues a batch (n = 0: drains instead); returns the number of frames of the batch whose results are ready (read them with
 * vmh_pipeline_result before the next call but one), 0 if none is, or a negative status */
int vmh_pipeline_submit(vmh_pipeline* p, int n, const vmh_mesh* const* meshes, const real* Hoc16s, const vmh_lens_t* lenses,
                        const void* const* images, const uint32_t* fourccs) {
    GUARD({
        if (n == 0) p->done = p->pipe->flush();
        else if (p->model == VMH_RING6) {
            std::vector<HipEngine::Frame<Ring6>> frames(n);
            for (int i = 0; i < n; ++i) {
                if (!meshes[i]->r6) throw std::invalid_argument("mesh model does not match the pipeline");
                frames[i] = HipEngine::Frame<Ring6>{meshes[i]->r6, to_hoc(Hoc16s + 16 * i), to_lens(lenses + i), images[i], fourccs[i]};
            }
            p->done = p->pipe->submit<Ring6>(frames);
        }
        else {
            std::vector<HipEngine::Frame<NMGrid8>> frames(n);
            for (int i = 0; i < n; ++i) {
                if (!meshes[i]->g8) throw std::invalid_argument("mesh model does not match the pipeline");
                frames[i] = HipEngine::Frame<NMGrid8>{meshes[i]->g8, to_hoc(Hoc16s + 16 * i), to_lens(lenses + i), images[i], fourccs[i]};
            }
            p->done = p->pipe->submit<NMGrid8>(frames);
        }
        return p->done ? int(p->done->size()) : 0;
    })
}
/* frame i of the ready batch: its visible count and the arrays (inside the pipeline's page-locked memory) */
int vmh_pipeline_result(vmh_pipeline* p, int i, real** px, int32_t** gidx, int32_t** nb, real** cls) {
    GUARD({
        if (!p->done) throw std::invalid_argument("pipeline_result: no batch is ready");
        const vmhip_result& r = p->done->at(size_t(i));
        *px = r.pixel_coordinates, *gidx = r.global_indices, *nb = r.neighbourhood, *cls = r.classifications;
        return r.capacity;
    })
}
int vmh_pipeline_n_classes(vmh_pipeline* p) { return p->pipe->engine(0).n_classes(); }
/* captures, graph launches and kernel-by-kernel launches of the pipeline's three engines together */
int vmh_pipeline_graph_stats(vmh_pipeline* p, int64_t* captures, int64_t* graph_launches, int64_t* eager_launches) {
    GUARD({
        const auto s = p->pipe->graph_stats();
        *captures = s.captures, *graph_launches = s.graph_launches, *eager_launches = s.eager_launches;
        return 0;
    })
}
#endif  // !VMH_DOUBLE
}

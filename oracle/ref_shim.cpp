/*
 * ref_shim.cpp - the oracle's C interface implemented by instantiating the reference's own headers.
 *
 * TEST INFRASTRUCTURE ONLY. Compiled only where the reference tree is mounted (the Makefile passes
 * -I$(REFERENCE)/cpp); nothing of the reference is copied. The output goes to _ref/libvm_ref.so (Scalar = float)
 * and, compiled with -DVMO_REAL=double, to _ref/libvm_ref_f64.so (Scalar = double). It is
 * used to prove that vm_oracle.cpp and the engine's host-side mesh code are bit-identical to the
 * reference, and may be timed as the CPU baseline of kind "reference".
 *
 * Every vmo_classify() call constructs a fresh cpu::Engine, because the reference engine never clears
 * its input buffer (engine/cpu/engine.hpp:196-206,303) and is only correct on its first call.
 */
#include <limits>
#include <stdexcept>
#include <string>
// the three includes above must come first: engine/cpu/bayer.hpp and pixel.hpp use std::runtime_error
// without including <stdexcept>, utility/math.hpp uses std::numeric_limits without <limits>
#include <cstring>
#include <map>
#include <memory>
#include <vector>

#include "visualmesh/engine/cpu/engine.hpp"
#include "visualmesh/geometry/Circle.hpp"
#include "visualmesh/geometry/Sphere.hpp"
#include "visualmesh/mesh.hpp"
#include "visualmesh/model/nmgrid8.hpp"
#include "visualmesh/model/ring6.hpp"
#include "visualmesh/visualmesh.hpp"
#include "vm_oracle.h"

typedef vmo_real real;

using visualmesh::Lens;
using visualmesh::Mesh;
using visualmesh::VisualMesh;
using visualmesh::geometry::Circle;
using visualmesh::geometry::Sphere;
using visualmesh::model::NMGrid8;
using visualmesh::model::Ring6;
typedef Mesh<real, Ring6> MeshR6;
typedef Mesh<real, NMGrid8> MeshG8;

struct vmo_mesh {
    const MeshR6* r6 = nullptr;
    const MeshG8* g8 = nullptr;
    std::unique_ptr<MeshR6> own_r6;
    std::unique_ptr<MeshG8> own_g8;
};

struct vmo_visualmesh {
    std::unique_ptr<VisualMesh<real, Ring6>> r6;
    std::unique_ptr<VisualMesh<real, NMGrid8>> g8;
    std::vector<real> heights;
    std::vector<std::unique_ptr<vmo_mesh>> views;
};

namespace {

Lens<real> to_lens(const vmo_lens* l) {
    Lens<real> lens;
    lens.dimensions = {{l->width, l->height}};
    lens.projection = visualmesh::LensProjection(l->projection);
    lens.focal_length = l->focal_length;
    lens.centre = {{l->centre[0], l->centre[1]}};
    lens.k = {{l->k[0], l->k[1]}};
    lens.fov = l->fov;
    return lens;
}
visualmesh::mat4<real> to_hoc(const real* H) {
    visualmesh::mat4<real> m;
    for (int i = 0; i < 4; ++i)
        for (int j = 0; j < 4; ++j) m[i][j] = H[i * 4 + j];
    return m;
}
visualmesh::NetworkStructure<real> to_network(const vmo_network* net) {
    visualmesh::NetworkStructure<real> s;
    if (!net) return s;
    int li = 0;
    for (int g = 0; g < net->n_groups; ++g) {
        s.emplace_back();
        for (int l = 0; l < net->group_sizes[g]; ++l, ++li) {
            const vmo_layer& L = net->layers[li];
            visualmesh::Layer<real> layer;
            layer.weights.assign(L.n_in, std::vector<real>(L.n_out));
            for (int t = 0; t < L.n_in; ++t)
                for (int j = 0; j < L.n_out; ++j) layer.weights[t][j] = L.weights[size_t(t) * L.n_out + j];
            layer.biases.assign(L.biases, L.biases + L.n_out);
            layer.activation = visualmesh::ActivationFunction(L.activation);
            s.back().push_back(layer);
        }
    }
    return s;
}

template <typename M>
void copy_nodes(const M& mesh, real* rays, int32_t* nbr) {
    const int nn = int(mesh.nodes[0].neighbours.size());
    for (size_t i = 0; i < mesh.nodes.size(); ++i) {
        if (rays)
            for (int c = 0; c < 3; ++c) rays[i * 3 + c] = mesh.nodes[i].ray[c];
        if (nbr)
            for (int t = 0; t < nn; ++t) nbr[i * nn + t] = mesh.nodes[i].neighbours[t];
    }
}

template <typename PM>
int export_projection(const PM& p, int cap, real* px, int32_t* nb, int32_t* gidx) {
    const int V = int(p.global_indices.size());
    if (V > cap) return VMO_ERR_CAPACITY;
    const int nn = p.neighbourhood.empty() ? 0 : int(p.neighbourhood[0].size());
    for (int i = 0; i < V; ++i) {
        px[2 * i] = p.pixel_coordinates[i][0];
        px[2 * i + 1] = p.pixel_coordinates[i][1];
        gidx[i] = p.global_indices[i];
    }
    for (size_t i = 0; i < p.neighbourhood.size(); ++i)
        for (int t = 0; t < nn; ++t) nb[i * nn + t] = p.neighbourhood[i][t];
    return V;
}

template <typename M>
int do_project(const M& mesh, const real* H, const vmo_lens* l, int cap, real* px, int32_t* nb, int32_t* gidx) {
    visualmesh::engine::cpu::Engine<real> engine;
    auto p = engine(mesh, to_hoc(H), to_lens(l));
    return export_projection(p, cap, px, nb, gidx);
}
template <typename M>
int do_classify(const M& mesh, const real* H, const vmo_lens* l, const void* image, uint32_t fourcc,
                const vmo_network* net, int cap, real* px, int32_t* nb, int32_t* gidx, real* cls) {
    visualmesh::engine::cpu::Engine<real> engine(to_network(net));  // fresh engine for every call
    auto c = engine(mesh, to_hoc(H), to_lens(l), image, fourcc);
    const int V = export_projection(c, cap, px, nb, gidx);
    if (V > 0) std::memcpy(cls, c.classifications.data(), sizeof(real) * c.classifications.size());
    return V;
}

template <typename S>
real shape_fn(const S& s, int which, real a, real b) {
    switch (which) {
        case 0: return s.phi(a, b);
        case 1: return s.n(a, b);
        case 2: return s.theta(a, b);
        case 3: return s.k(a, b);
        default: return s.c();
    }
}

}  // namespace

extern "C" {

const char* vmo_name(void) { return "reference"; }

vmo_mesh* vmo_mesh_create(int model, int shape, real radius, real h, real k, real max_distance) {
    try {
        std::unique_ptr<vmo_mesh> m(new vmo_mesh());
        if (model == VMO_MODEL_RING6) {
            if (shape == VMO_SHAPE_SPHERE) m->own_r6.reset(new MeshR6(Sphere<real>(radius), h, k, max_distance));
            else if (shape == VMO_SHAPE_CIRCLE) m->own_r6.reset(new MeshR6(Circle<real>(radius), h, k, max_distance));
            else return nullptr;
            m->r6 = m->own_r6.get();
        }
        else if (model == VMO_MODEL_NMGRID8) {
            if (shape == VMO_SHAPE_SPHERE) m->own_g8.reset(new MeshG8(Sphere<real>(radius), h, k, max_distance));
            else if (shape == VMO_SHAPE_CIRCLE) m->own_g8.reset(new MeshG8(Circle<real>(radius), h, k, max_distance));
            else return nullptr;
            m->g8 = m->own_g8.get();
        }
        else return nullptr;
        return m.release();
    } catch (...) { return nullptr; }
}
void vmo_mesh_destroy(vmo_mesh* m) { delete m; }
int vmo_mesh_n_nodes(const vmo_mesh* m) { return m->r6 ? int(m->r6->nodes.size()) : int(m->g8->nodes.size()); }
int vmo_mesh_n_neighbours(const vmo_mesh* m) { return m->r6 ? 6 : 8; }
real vmo_mesh_h(const vmo_mesh* m) { return m->r6 ? m->r6->h : m->g8->h; }
void vmo_mesh_copy(const vmo_mesh* m, real* rays, int32_t* neighbours) {
    if (m->r6) copy_nodes(*m->r6, rays, neighbours);
    else copy_nodes(*m->g8, rays, neighbours);
}
int vmo_mesh_lookup(const vmo_mesh* m, const real* Hoc16, const vmo_lens* lens, int32_t* ranges, int cap) {
    try {
        const auto r = m->r6 ? m->r6->lookup(to_hoc(Hoc16), to_lens(lens)) : m->g8->lookup(to_hoc(Hoc16), to_lens(lens));
        for (int i = 0; i < int(r.size()) && i < cap; ++i) {
            ranges[2 * i] = r[i].first;
            ranges[2 * i + 1] = r[i].second;
        }
        return int(r.size());
    } catch (...) { return VMO_ERR_LENS; }
}

vmo_visualmesh* vmo_visualmesh_create(int model, int shape, real radius, real min_h, real max_h, real k,
                                      real max_error, real max_distance) {
    try {
        std::unique_ptr<vmo_visualmesh> v(new vmo_visualmesh());
        if (model == VMO_MODEL_RING6) {
            if (shape == VMO_SHAPE_SPHERE)
                v->r6.reset(new VisualMesh<real, Ring6>(Sphere<real>(radius), min_h, max_h, k, max_error, max_distance));
            else
                v->r6.reset(new VisualMesh<real, Ring6>(Circle<real>(radius), min_h, max_h, k, max_error, max_distance));
        }
        else if (model == VMO_MODEL_NMGRID8) {
            if (shape == VMO_SHAPE_SPHERE)
                v->g8.reset(new VisualMesh<real, NMGrid8>(Sphere<real>(radius), min_h, max_h, k, max_error, max_distance));
            else
                v->g8.reset(new VisualMesh<real, NMGrid8>(Circle<real>(radius), min_h, max_h, k, max_error, max_distance));
        }
        else return nullptr;
        /* The LUT map is private; enumerate the meshes by probing height() between distinct answers.
         * Every mesh's own h is a key, so walking upward from min_h by asking for "just above the last
         * key's midpoint" finds each one: instead, probe a fine grid and collect distinct h values. */
        std::map<real, const void*> found;
        const int steps = 200000;
        for (int i = 0; i <= steps; ++i) {
            const real q = min_h + (max_h - min_h) * (real(i) / real(steps));
            if (v->r6) {
                const MeshR6& mm = v->r6->height(q);
                found[mm.h] = &mm;
            }
            else {
                const MeshG8& mm = v->g8->height(q);
                found[mm.h] = &mm;
            }
        }
        for (auto& kv : found) {
            v->heights.push_back(kv.first);
            std::unique_ptr<vmo_mesh> view(new vmo_mesh());
            if (v->r6) view->r6 = static_cast<const MeshR6*>(kv.second);
            else view->g8 = static_cast<const MeshG8*>(kv.second);
            v->views.push_back(std::move(view));
        }
        return v.release();
    } catch (...) { return nullptr; }
}
void vmo_visualmesh_destroy(vmo_visualmesh* v) { delete v; }
int vmo_visualmesh_n_meshes(const vmo_visualmesh* v) { return int(v->views.size()); }
const vmo_mesh* vmo_visualmesh_mesh(const vmo_visualmesh* v, int i) { return v->views[i].get(); }
const vmo_mesh* vmo_visualmesh_height(const vmo_visualmesh* v, real h) {
    const real key = v->r6 ? v->r6->height(h).h : v->g8->height(h).h;
    for (size_t i = 0; i < v->heights.size(); ++i)
        if (v->heights[i] == key) return v->views[i].get();
    return nullptr;
}

int vmo_project(const vmo_mesh* m, const real* Hoc16, const vmo_lens* lens, int cap, real* px, int32_t* nb,
                int32_t* gidx) {
    try {
        return m->r6 ? do_project(*m->r6, Hoc16, lens, cap, px, nb, gidx) : do_project(*m->g8, Hoc16, lens, cap, px, nb, gidx);
    } catch (...) { return VMO_ERR_LENS; }
}
int vmo_classify(const vmo_mesh* m, const real* Hoc16, const vmo_lens* lens, const void* image, uint32_t fourcc,
                 const vmo_network* net, int cap, real* px, int32_t* nb, int32_t* gidx, real* cls) {
    try {
        return m->r6 ? do_classify(*m->r6, Hoc16, lens, image, fourcc, net, cap, px, nb, gidx, cls)
                     : do_classify(*m->g8, Hoc16, lens, image, fourcc, net, cap, px, nb, gidx, cls);
    } catch (const std::runtime_error& e) {
        return std::string(e.what()).find("format") != std::string::npos
                   || std::string(e.what()).find("bayer") != std::string::npos
                 ? VMO_ERR_FORMAT
                 : VMO_ERR_LENS;
    } catch (...) { return VMO_ERR_LENS; }
}

void vmo_fn_project(const real* r, const vmo_lens* lens, real* px2) {
    const auto p = visualmesh::project(visualmesh::vec3<real>{{r[0], r[1], r[2]}}, to_lens(lens));
    px2[0] = p[0], px2[1] = p[1];
}
void vmo_fn_unproject(const real* px2, const vmo_lens* lens, real* ray3) {
    const auto r = visualmesh::unproject(visualmesh::vec2<real>{{px2[0], px2[1]}}, to_lens(lens));
    ray3[0] = r[0], ray3[1] = r[1], ray3[2] = r[2];
}
int vmo_fn_interpolate(const real* px2, const void* image, int width, int height, uint32_t fourcc, real* out4) {
    try {
        const auto v = visualmesh::engine::cpu::interpolate(visualmesh::vec2<real>{{px2[0], px2[1]}},
                                                            reinterpret_cast<const uint8_t*>(image),
                                                            visualmesh::vec2<int>{{width, height}}, fourcc);
        for (int i = 0; i < 4; ++i) out4[i] = v[i];
        return VMO_OK;
    } catch (...) { return VMO_ERR_FORMAT; }
}
int vmo_fn_get_pixel(int x, int y, const void* image, int width, int height, uint32_t fourcc, real* out4) {
    try {
        const auto v = visualmesh::engine::cpu::get_pixel<real>(visualmesh::vec2<int>{{x, y}},
                                                                 reinterpret_cast<const uint8_t*>(image),
                                                                 visualmesh::vec2<int>{{width, height}}, fourcc);
        for (int i = 0; i < 4; ++i) out4[i] = v[i];
        return VMO_OK;
    } catch (...) { return VMO_ERR_FORMAT; }
}
void vmo_fn_activation(int activation, real* data, int n_rows, int dims) {
    std::vector<real> v(data, data + size_t(n_rows) * dims);
    visualmesh::engine::cpu::apply_activation(visualmesh::ActivationFunction(activation), v, dims);
    std::memcpy(data, v.data(), sizeof(real) * v.size());
}
real vmo_fn_shape(int shape, real radius, int which, real a, real b) {
    if (shape == VMO_SHAPE_SPHERE) return shape_fn(Sphere<real>(radius), which, a, b);
    return shape_fn(Circle<real>(radius), which, a, b);
}
void vmo_fn_libm(int which, const real* x, real* y, int n) {
    for (int i = 0; i < n; ++i)
        y[i] = which == 0 ? std::acos(x[i]) : which == 1 ? std::sin(x[i]) : which == 2 ? std::tan(x[i]) : std::sqrt(x[i]);
}
}

/*
 * vm_oracle.h - C interface of the CPU oracle for the Visual Mesh inference path.
 *
 * TEST INFRASTRUCTURE ONLY. This library restates, on the CPU and in fp32, what the reference CPU
 * engine computes (mesh generation, BSP lookup, projection, sampling, graph convolution). It exists
 * to check the HIP engine and to be timed as the CPU baseline. Nothing in the shipped engine may
 * link, load or call it.
 *
 * The same interface is implemented twice:
 *   libvm_oracle.so      - the restatement in vm_oracle.cpp (travels everywhere)
 *   _ref/libvm_ref.so    - ref_shim.cpp, a thin wrapper that instantiates the reference's own
 *                          headers (only buildable where the reference tree is mounted)
 * so that one test harness can compare restatement, reference and HIP engine.
 */
#ifndef VM_ORACLE_H
#define VM_ORACLE_H

#include <stdint.h>

/* The reference's engines and meshes are templates over Scalar (engine/cpu/engine.hpp:49-50, mesh.hpp:56); this
 * interface is compiled once per Scalar: vmo_real is float in libvm_oracle.so and _ref/libvm_ref.so, double (built with
 * -DVMO_REAL=double) in libvm_oracle_f64.so and _ref/libvm_ref_f64.so. */
#ifndef VMO_REAL
#define VMO_REAL float
#endif
typedef VMO_REAL vmo_real;

#ifdef __cplusplus
extern "C" {
#endif

enum { VMO_MODEL_RING6 = 0, VMO_MODEL_NMGRID8 = 1 };
enum { VMO_SHAPE_SPHERE = 0, VMO_SHAPE_CIRCLE = 1 };
/* Same numbering as the reference's LensProjection (lens.hpp:33) and ActivationFunction
 * (network_structure.hpp:34-39). */
enum { VMO_RECTILINEAR = 0, VMO_EQUISOLID = 1, VMO_EQUIDISTANT = 2 };
enum { VMO_SELU = 0, VMO_RELU = 1, VMO_SOFTMAX = 2, VMO_TANH = 3 };

enum { VMO_OK = 0, VMO_ERR_FORMAT = -2, VMO_ERR_LENS = -3, VMO_ERR_ARG = -4, VMO_ERR_CAPACITY = -5 };

typedef struct vmo_lens {
    int32_t width, height;
    int32_t projection;
    vmo_real focal_length;
    vmo_real centre[2];
    vmo_real k[2];
    vmo_real fov;
} vmo_lens;

/* One dense layer: weights[n_in][n_out] row-major (the layout model.yaml and NetworkStructure use),
 * biases[n_out]. */
typedef struct vmo_layer {
    int32_t n_in, n_out;
    int32_t activation;
    const vmo_real* weights;
    const vmo_real* biases;
} vmo_layer;

/* A network is n_groups convolutional groups; group g owns group_sizes[g] consecutive layers. */
typedef struct vmo_network {
    int32_t n_groups;
    const int32_t* group_sizes;
    const vmo_layer* layers;
} vmo_network;

typedef struct vmo_mesh vmo_mesh;
typedef struct vmo_visualmesh vmo_visualmesh;

const char* vmo_name(void); /* "oracle" or "reference" */

/* ---- mesh (host side of the path) ---- */
vmo_mesh* vmo_mesh_create(int model, int shape, vmo_real radius, vmo_real h, vmo_real k, vmo_real max_distance);
void vmo_mesh_destroy(vmo_mesh* m);
int vmo_mesh_n_nodes(const vmo_mesh* m);
int vmo_mesh_n_neighbours(const vmo_mesh* m);
vmo_real vmo_mesh_h(const vmo_mesh* m);
/* rays[n_nodes][3], neighbours[n_nodes][n_neighbours] */
void vmo_mesh_copy(const vmo_mesh* m, vmo_real* rays, int32_t* neighbours);
/* Writes up to cap (first,second) pairs, returns the number of ranges found. */
int vmo_mesh_lookup(const vmo_mesh* m, const vmo_real* Hoc16, const vmo_lens* lens, int32_t* ranges, int cap);

vmo_visualmesh* vmo_visualmesh_create(int model, int shape, vmo_real radius, vmo_real min_h, vmo_real max_h, vmo_real k,
                                      vmo_real max_error, vmo_real max_distance);
void vmo_visualmesh_destroy(vmo_visualmesh* v);
int vmo_visualmesh_n_meshes(const vmo_visualmesh* v);
/* i-th mesh in ascending height order (borrowed) */
const vmo_mesh* vmo_visualmesh_mesh(const vmo_visualmesh* v, int i);
/* the mesh VisualMesh::height(h) selects (borrowed) */
const vmo_mesh* vmo_visualmesh_height(const vmo_visualmesh* v, vmo_real h);

/* ---- engine ---- */
/* ProjectedMesh. Buffers: px[cap][2], gidx[cap], nb[cap+1][n_neighbours]. Returns V (visible nodes) or a
 * negative error. cap must be at least the number of candidates in the lookup ranges;
 * vmo_mesh_n_nodes() is always enough. */
int vmo_project(const vmo_mesh* m, const vmo_real* Hoc16, const vmo_lens* lens, int cap, vmo_real* px, int32_t* nb,
                int32_t* gidx);
/* ClassifiedMesh, computed with a fresh engine state on every call. cls[(cap+1) * n_out_last]. If the
 * network has no groups the sampled 4-channel input (plus null row) is returned, as in the reference. If
 * nothing is visible returns 0 and writes nothing (default-constructed result). */
int vmo_classify(const vmo_mesh* m, const vmo_real* Hoc16, const vmo_lens* lens, const void* image, uint32_t fourcc,
                 const vmo_network* net, int cap, vmo_real* px, int32_t* nb, int32_t* gidx, vmo_real* cls);

/* ---- single functions, exposed so tests can pin each one separately ---- */
void vmo_fn_project(const vmo_real* cam_ray3, const vmo_lens* lens, vmo_real* px2);
void vmo_fn_unproject(const vmo_real* px2, const vmo_lens* lens, vmo_real* ray3);
int vmo_fn_interpolate(const vmo_real* px2, const void* image, int width, int height, uint32_t fourcc, vmo_real* out4);
int vmo_fn_get_pixel(int x, int y, const void* image, int width, int height, uint32_t fourcc, vmo_real* out4);
void vmo_fn_activation(int activation, vmo_real* data, int n_rows, int dims);
/* shape functions: which = 0 phi(n,h), 1 n(phi,h), 2 theta(n,h), 3 k(h0,h1), 4 c() */
vmo_real vmo_fn_shape(int shape, vmo_real radius, int which, vmo_real a, vmo_real b);
/* the host C library functions the lens projection is built from: which = 0 acos, 1 sin, 2 tan, 3 sqrt of vmo_real */
void vmo_fn_libm(int which, const vmo_real* x, vmo_real* y, int n);

#ifdef __cplusplus
}
#endif
#endif

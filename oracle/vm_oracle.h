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
    float focal_length;
    float centre[2];
    float k[2];
    float fov;
} vmo_lens;

/* One dense layer: weights[n_in][n_out] row-major (the layout model.yaml and NetworkStructure use),
 * biases[n_out]. */
typedef struct vmo_layer {
    int32_t n_in, n_out;
    int32_t activation;
    const float* weights;
    const float* biases;
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
vmo_mesh* vmo_mesh_create(int model, int shape, float radius, float h, float k, float max_distance);
void vmo_mesh_destroy(vmo_mesh* m);
int vmo_mesh_n_nodes(const vmo_mesh* m);
int vmo_mesh_n_neighbours(const vmo_mesh* m);
float vmo_mesh_h(const vmo_mesh* m);
/* rays[n_nodes][3], neighbours[n_nodes][n_neighbours] */
void vmo_mesh_copy(const vmo_mesh* m, float* rays, int32_t* neighbours);
/* Writes up to cap (first,second) pairs, returns the number of ranges found. */
int vmo_mesh_lookup(const vmo_mesh* m, const float* Hoc16, const vmo_lens* lens, int32_t* ranges, int cap);

vmo_visualmesh* vmo_visualmesh_create(int model, int shape, float radius, float min_h, float max_h, float k,
                                      float max_error, float max_distance);
void vmo_visualmesh_destroy(vmo_visualmesh* v);
int vmo_visualmesh_n_meshes(const vmo_visualmesh* v);
/* i-th mesh in ascending height order (borrowed) */
const vmo_mesh* vmo_visualmesh_mesh(const vmo_visualmesh* v, int i);
/* the mesh VisualMesh::height(h) selects (borrowed) */
const vmo_mesh* vmo_visualmesh_height(const vmo_visualmesh* v, float h);

/* ---- engine ---- */
/* ProjectedMesh. Buffers: px[cap][2], gidx[cap], nb[cap+1][n_neighbours]. Returns V (visible nodes) or a
 * negative error. cap must be at least the number of candidates in the lookup ranges;
 * vmo_mesh_n_nodes() is always enough. */
int vmo_project(const vmo_mesh* m, const float* Hoc16, const vmo_lens* lens, int cap, float* px, int32_t* nb,
                int32_t* gidx);
/* ClassifiedMesh, computed with a fresh engine state on every call. cls[(cap+1) * n_out_last]. If the
 * network has no groups the sampled 4-channel input (plus null row) is returned, as in the reference. If
 * nothing is visible returns 0 and writes nothing (default-constructed result). */
int vmo_classify(const vmo_mesh* m, const float* Hoc16, const vmo_lens* lens, const void* image, uint32_t fourcc,
                 const vmo_network* net, int cap, float* px, int32_t* nb, int32_t* gidx, float* cls);

/* ---- single functions, exposed so tests can pin each one separately ---- */
void vmo_fn_project(const float* cam_ray3, const vmo_lens* lens, float* px2);
void vmo_fn_unproject(const float* px2, const vmo_lens* lens, float* ray3);
int vmo_fn_interpolate(const float* px2, const void* image, int width, int height, uint32_t fourcc, float* out4);
int vmo_fn_get_pixel(int x, int y, const void* image, int width, int height, uint32_t fourcc, float* out4);
void vmo_fn_activation(int activation, float* data, int n_rows, int dims);
/* shape functions: which = 0 phi(n,h), 1 n(phi,h), 2 theta(n,h), 3 k(h0,h1), 4 c() */
float vmo_fn_shape(int shape, float radius, int which, float a, float b);
/* the host C library functions the lens projection is built from: which = 0 acosf, 1 sinf, 2 tanf, 3 sqrtf */
void vmo_fn_libm(int which, const float* x, float* y, int n);

#ifdef __cplusplus
}
#endif
#endif

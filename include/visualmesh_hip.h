/*
 * visualmesh_hip.h - C ABI of libvisualmesh_hip.so, the MI355X (gfx950) back end of
 * visualmesh::engine::hip::Engine.
 *
 * The library owns all HIP state. Callers pass plain host pointers and sizes; there are no C++ or
 * framework types in any signature. All functions return VMHIP_OK (0) or a negative status;
 * vmhip_last_error() returns the message of the last failure on the calling thread.
 *
 * What stays with the caller (host C++): mesh generation and the BSP range lookup
 * (reference cpp/visualmesh/mesh.hpp:424-467 and :499-595). The caller hands over the mesh's node
 * table once (vmhip_mesh_upload) and, per frame, the index ranges that lookup returned.
 *
 * What the library replaces, per frame (reference cpp/visualmesh/engine/cpu/engine.hpp):
 *   :97-125   projection of every candidate node, strict on-screen filter, order-preserving compaction
 *   :127-143  reverse lookup and local neighbourhood table, null row last
 *   :198-206  image sampling (pixel.hpp:43-144, bayer.hpp:95-158) and the (-1,-1,-1,-1) null row
 *   :213-264  per convolutional group: neighbour gather + dense layers + activation
 *   :267-272  result assembly
 *
 * Threading: like the reference engines, an engine (and every batch made from it) is used from one
 * thread at a time. Meshes are immutable and may be shared by engines on different threads.
 */
#ifndef VISUALMESH_HIP_H
#define VISUALMESH_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
    VMHIP_OK = 0,
    VMHIP_ERR_HIP = -1,      /* a HIP runtime call failed (no device, out of memory, launch failure) */
    VMHIP_ERR_FORMAT = -2,   /* unsupported fourcc: reference engine/cpu/pixel.hpp:100 throws here */
    VMHIP_ERR_LENS = -3,     /* unknown lens projection: reference utility/projection.hpp:174 throws */
    VMHIP_ERR_ARGUMENT = -4, /* null pointer, inconsistent sizes, network does not fit the mesh */
    VMHIP_ERR_CAPACITY = -5  /* a caller-provided result buffer is too small */
};

/* Same numbering as the reference's LensProjection (lens.hpp:33). */
enum { VMHIP_RECTILINEAR = 0, VMHIP_EQUISOLID = 1, VMHIP_EQUIDISTANT = 2 };
/* Same numbering as the reference's ActivationFunction (network_structure.hpp:34-39). */
enum { VMHIP_SELU = 0, VMHIP_RELU = 1, VMHIP_SOFTMAX = 2, VMHIP_TANH = 3 };
/* Arithmetic of the graph-convolution layers of a float engine (vmhip_engine_create); its projection and sampling are
 * always fp32. VMHIP_FP64 names the arithmetic of the double engines further down, which have entry points of their own
 * (every number they take or return is a double, so the structures differ): vmhip_engine_create refuses it and says so. */
enum { VMHIP_FP32 = 0, VMHIP_BF16 = 1, VMHIP_FP64 = 2, VMHIP_SPLIT = 3 };
/* VMHIP_BF16: layers that are 64 wide on both sides run on the bf16 matrix instructions, with rows between them stored as
 * bf16 or as pairs of bf16 (probabilities within 1e-2 of the fp32 result; the other layers stay fp32).
 * VMHIP_SPLIT: the same layers on the same instructions, but every row between them as pairs of bf16 (a value's leading
 * 8 bits and the bf16 of what they leave over) and three products per pair of values. Probabilities stay within 1e-4
 * of the CPU engine's (fp32's parity bar) for networks of up to six such layers - 2.6e-5 at most on the 6 x 64 network
 * at full size, 3.4e-5 on other seeds - and within 2e-4 for up to ten (9.7e-5 measured on one seed: no margin against
 * 1e-4); what the pairs leave out adds up with depth, so an engine with more than ten such layers is refused
 * (VMHIP_ERR_ARGUMENT): use VMHIP_FP32 there. More than twice the fp32 engine's speed on such networks, more than the
 * fp32 matrix peak would allow. The measurement overrides VMHIP_BF16_ROUNDED / VMHIP_BF16_ROUNDED_AT are ignored for
 * this precision: its contract has no bf16-rounded row. */

/* POD mirror of visualmesh::Lens<float> (reference lens.hpp:41-52). */
typedef struct vmhip_lens {
    int32_t width, height; /* dimensions[0], dimensions[1] */
    int32_t projection;
    float focal_length; /* pixels */
    float centre[2];
    float k[2];
    float fov; /* radians, full angle */
} vmhip_lens;

/* One dense layer (reference network_structure.hpp:43-47): weights[n_in][n_out] row major, the layout
 * of NetworkStructure and model.yaml, biases[n_out]. */
typedef struct vmhip_layer {
    int32_t n_in, n_out;
    int32_t activation;
    const float* weights;
    const float* biases;
} vmhip_layer;

/* NetworkStructure flattened: n_groups convolutional groups, group g owning group_sizes[g] consecutive
 * entries of layers. The first layer of a group consumes (n_neighbours+1) * width_of_previous_output
 * values (4 for the first group), ordered [self, neighbour 0, ..., neighbour n-1]
 * (reference engine/cpu/engine.hpp:222-231). */
typedef struct vmhip_network {
    int32_t n_groups;
    const int32_t* group_sizes;
    const vmhip_layer* layers;
} vmhip_network;

/* Inputs of one frame. */
/* Lookup on the device instead of on the host (the reference walks its BSP on the host, mesh.hpp:499-595): the
 * mesh carries its cone tree (vmhip_mesh_attach_tree), a frame names what the walk compares against, and
 * vmhip_batch_stage works out the frame's ranges itself. The host side of the engine fills this in
 * (cpp/visualmesh/detail/cone_tree.hpp: lookup_parameters). */
typedef struct vmhip_tree_element {
    int32_t first, last; /* node range [first, last) of the element */
    int32_t child[2];    /* -1, -1 for a leaf */
    float axis[3];       /* bounding cone of the element's nodes: axis, */
    float c, s;          /* cosine and sine of its half angle */
} vmhip_tree_element;
typedef struct vmhip_lookup {
    float cos_half_fov, sin_half_fov;
    float edge[4][5];    /* cones hugging the four screen edges, in observation-plane space: axis, cosine, sine */
} vmhip_lookup;

typedef struct vmhip_frame {
    const struct vmhip_mesh* mesh;
    float Rco[9];          /* row major; Rco[i][j] = Hoc[j][i] (reference engine/cpu/engine.hpp:95) */
    vmhip_lens lens;
    const int32_t* ranges; /* n_ranges pairs (first, one-past-last), ascending and disjoint: Mesh::lookup's output */
    int32_t n_ranges;
    const void* image;     /* tightly packed rows, width*height*bytes_per_pixel(fourcc) bytes; NULL when only projecting */
    uint32_t fourcc;       /* little-endian four character code (reference utility/fourcc.hpp:34-36) */
    const vmhip_lookup* lookup; /* not NULL: ranges / n_ranges are ignored and the lookup runs on the device */
} vmhip_frame;

/* Outputs of one frame, in caller-owned buffers. capacity counts nodes: it must be at least the number
 * of candidate nodes (the sum of the range lengths). n_visible is written by the library.
 *   pixel_coordinates [capacity][2]              first n_visible rows valid
 *   global_indices    [capacity]                 first n_visible valid, ascending
 *   neighbourhood     [capacity+1][n_neighbours] first n_visible+1 rows valid, last one is the null row
 *   classifications   [capacity+1][n_classes]    first n_visible+1 rows valid; may be NULL when projecting
 * Any pointer may be NULL to skip that output. If nothing is visible n_visible is 0 and nothing is
 * written (the reference returns a default-constructed result, engine/cpu/engine.hpp:193). */
typedef struct vmhip_result {
    int32_t capacity;
    int32_t n_visible;
    float* pixel_coordinates;
    int32_t* global_indices;
    int32_t* neighbourhood;
    float* classifications;
} vmhip_result;

typedef struct vmhip_engine vmhip_engine;
typedef struct vmhip_mesh vmhip_mesh;
typedef struct vmhip_batch vmhip_batch;

const char* vmhip_last_error(void);

/* Replaces the engine constructor (reference engine/cpu/engine.hpp:57-71, engine/opencl/engine.hpp:189):
 * validates the network, converts the weights to the kernels' layouts and uploads them. net may have
 * zero groups (projection only, or classification returning the sampled 4-channel input). */
int vmhip_engine_create(const vmhip_network* net, int32_t n_neighbours, int32_t precision, vmhip_engine** out);
void vmhip_engine_destroy(vmhip_engine* engine);
/* Width of the classification rows this engine produces (4 for an empty network). */
int32_t vmhip_engine_n_classes(const vmhip_engine* engine);

/* Replaces the per-mesh device cache of the reference's OpenCL engine (engine/opencl/engine.hpp:603-625):
 * rays[n_nodes][3] and neighbours[n_nodes][n_neighbours] (global indices, n_nodes = "no neighbour") are
 * copied to the device once. The handle is independent of any engine. */
int vmhip_mesh_upload(const float* rays, const int32_t* neighbours, int32_t n_nodes, int32_t n_neighbours,
                      vmhip_mesh** out);
void vmhip_mesh_release(vmhip_mesh* mesh);
/* copies the mesh's cone tree (element 0 is the root) to the device, for frames that ask for the lookup there */
int vmhip_mesh_attach_tree(vmhip_mesh* mesh, const vmhip_tree_element* elements, int32_t n_elements);

/* Page-locked host memory for images (and result arrays): copies between it and the device run at the link's full
 * rate and do not hold the caller up, copies from ordinary memory are staged through small buffers by the runtime.
 * No counterpart in the reference, which leaves image memory to its caller (engine/opencl/engine.hpp:307-315 copies
 * from whatever pointer it is given). NULL if the allocation fails. */
void* vmhip_host_alloc(size_t bytes);
void vmhip_host_free(void* memory);

/* Replaces cpu::Engine::operator()(mesh, Hoc, lens) (reference engine/cpu/engine.hpp:84-147). */
int vmhip_project(vmhip_engine* engine, const vmhip_frame* frame, vmhip_result* result);
/* Replaces cpu::Engine::operator()(mesh, Hoc, lens, image, format) (reference engine/cpu/engine.hpp:180-273). */
int vmhip_classify(vmhip_engine* engine, const vmhip_frame* frame, vmhip_result* result);
/* The same for n_frames independent frames in one pass (the reference has no batched call; its
 * benchmark loops over frames, example/benchmark.cpp:50-58). Frames may use different meshes and lenses. */
int vmhip_classify_batch(vmhip_engine* engine, const vmhip_frame* frames, int32_t n_frames, vmhip_result* results);

/* Staged form of vmhip_classify_batch for pipelines that keep frames resident on the device:
 *   stage  copies the frames' inputs to the device (images, poses, lenses, ranges) and sizes the workspace
 *   run    executes the whole path on the device and waits for it; may be repeated
 *   fetch  copies the results of the last run into caller buffers
 * classify != 0 runs sampling and the network, 0 stops after the neighbourhood table. */
int vmhip_batch_create(vmhip_engine* engine, vmhip_batch** out);
void vmhip_batch_destroy(vmhip_batch* batch);
int vmhip_batch_stage(vmhip_batch* batch, const vmhip_frame* frames, int32_t n_frames, int32_t classify);
/* vmhip_batch_stage without the wait for its copies: they are queued on the engine's stream ahead of the run and the call
 * returns, so a caller that rotates engines (one staging, one running, one copying out) is not held up for the 2 ms
 * that 84 MB of images take to cross the bus. The frames' images must be page-locked (vmhip_host_alloc) for the copies
 * to run on their own, and must stay untouched until the batch's next vmhip_batch_run or vmhip_batch_wait has returned.
 * No counterpart in the reference, whose OpenCL engine copies the image inside the call (engine/opencl/engine.hpp:307-315). */
int vmhip_batch_stage_async(vmhip_batch* batch, const vmhip_frame* frames, int32_t n_frames, int32_t classify);
/* The lookup ranges of a staged frame, as pairs (first, one-past-last): the caller's own, or what the lookup on the
 * device produced. Returns their number (ranges may be NULL to ask for it only) or a negative status. */
int vmhip_batch_ranges(const vmhip_batch* batch, int32_t frame, int32_t* ranges, int32_t capacity);

/* Replaces the LookupVisualMesh op of the training pipeline (reference tensorflow/lookup.cpp:186-249) for the frames of
 * a staged batch (no run needed): per frame, for every node of its lookup ranges in order,
 *   vectors [capacity][3]               the node's unit vector (the op's output "vectors")
 *   graph   [capacity][n_neighbours+1]  its own position, then its neighbours' positions along the ranges (the op's
 *                                       output "neighbours"); a neighbour outside the ranges is INT32_MIN with
 *                                       VMHIP_EDGE_HARD and the node's own position with VMHIP_EDGE_SAME
 *                                       (training/dataset/projection/visual_mesh.py:82-89)
 *   pixels  [capacity][2]               (x, y) as vmhip_project computes them, on screen or not; may be NULL
 * n_points is written by the library; capacity must be at least the sum of the frame's range lengths. */
enum { VMHIP_EDGE_HARD = 0, VMHIP_EDGE_SAME = 1 };
typedef struct vmhip_lookup_export {
    int32_t capacity;
    int32_t n_points;
    float* vectors;
    int32_t* graph;
    float* pixels;
} vmhip_lookup_export;
int vmhip_batch_export(vmhip_batch* batch, int32_t edge_type, vmhip_lookup_export* per_frame);
int vmhip_batch_run(vmhip_batch* batch);
/* The two halves of vmhip_batch_run: run_async puts the pass on the engine's stream and returns, wait blocks until it
 * is done (and settles the screen-edge decisions with the host, as run does). Between the two the caller is free,
 * e.g. to stage the next frames into a batch of another engine, whose copies then overlap this pass. Counts, fetch
 * and detect need the wait; the batch must not be staged or run again before it. */
int vmhip_batch_run_async(vmhip_batch* batch);
int vmhip_batch_wait(vmhip_batch* batch);
/* How the passes of a batch object were put on the stream since it was made: passes captured into a HIP graph
 * (captures), passes launched as a replay of a captured graph (graph_launches, the capturing pass included) and passes
 * launched kernel by kernel (eager_launches). A captured pass holds addresses, launch grids and the number of frames
 * only - the tiles in use, the frame descriptions and the range and tile tables are read from device memory - so it
 * outlives the batch it was captured with: staging other frames keeps it, and it is captured again only when a device
 * buffer had to grow, a batch needs larger grids or has another number of frames, or the profiling mode changes. This
 * is what the reference's OpenCL engine does with its kernels and grow-only buffers, re-issued per frame with new
 * arguments (engine/opencl/engine.hpp:455-489, :740-835). Any pointer may be NULL. */
int vmhip_batch_graph_stats(const vmhip_batch* batch, int64_t* captures, int64_t* graph_launches, int64_t* eager_launches);
/* n_visible[n_frames] of the last run */
int vmhip_batch_counts(const vmhip_batch* batch, int32_t* n_visible);
int vmhip_batch_fetch(vmhip_batch* batch, vmhip_result* results);
/* The two halves of vmhip_batch_fetch: fetch_async queues the copies on the engine's stream and returns (n_visible is
 * already written), fetch_wait blocks until they are done. With result arrays from vmhip_host_alloc the copies run
 * while the caller stages the next frames into another engine's batch, on the bus's other direction; into ordinary
 * memory they are not asynchronous. Between the two the batch must not be staged, run, read or exported, and the
 * arrays must not be touched. */
int vmhip_batch_fetch_async(vmhip_batch* batch, vmhip_result* results);
int vmhip_batch_fetch_wait(vmhip_batch* batch);
/* vmhip_batch_fetch_async as one transfer: a kernel gathers the arrays of all frames into one block on the device and a
 * single copy brings it into `block` (page-locked memory from vmhip_host_alloc, at least vmhip_batch_fetch_packed_size()
 * bytes, which is known once the run has been waited for); results[i] is filled in by the library with n_visible,
 * capacity = n_visible and pointers into `block` (NULL for a frame that sees nothing, and for classifications after a
 * projection-only run). 64 copies of 0.8 MB on average become one of 50 MB for a 16-frame batch, which crosses the bus in
 * two thirds of the time. Finished by vmhip_batch_fetch_wait like vmhip_batch_fetch_async. No counterpart in the
 * reference. */
size_t vmhip_batch_fetch_packed_size(const vmhip_batch* batch);
int vmhip_batch_fetch_packed_async(vmhip_batch* batch, void* block, size_t bytes, vmhip_result* results);

/* vmhip_project for callers that cannot allocate: code under HIP graph capture, serving loops that must not call
 * hipMalloc, harnesses that forbid it. No counterpart in the reference. The call only launches kernels on hip_stream
 * (a hipStream_t, NULL = the default stream) and returns without waiting: no allocation, no copy, no wait.
 * Every pointer below is read or written by the device, so it must be device memory or memory from vmhip_host_alloc.
 *   ranges        n_ranges pairs (first, one-past-last) as Mesh::lookup returns them
 *   n_candidates  the sum of the range lengths (the launch grids are sized from it); capacity >= n_candidates
 *   n_visible     one word: the visible count, or -1 if the device found the pairs not ascending, not disjoint, outside
 *                 the mesh or not summing to n_candidates (then nothing else is written)
 *   pixel_coordinates [capacity][2], global_indices [capacity], neighbourhood [capacity+1][n_neighbours]
 *                 as in vmhip_result; all four are required. With visible nodes the null row follows them.
 * The workspace is one array of fixed size inside the library (11.3 MB per device, held until the process ends), so
 * sizes are limited as below and VMHIP_ERR_CAPACITY says which limit a call exceeds; calls that overlap on one
 * device race on that array, calls on one stream do not. The on-screen decisions are the device's own: they equal the
 * host's bit for bit where the host's C library is the one the device arithmetic reproduces (glibc's), and the
 * re-decision of near-edge nodes on the host that vmhip_project adds for other C libraries is not made here. */
enum {
    VMHIP_NOALLOC_MAX_CANDIDATES = 524288,
    VMHIP_NOALLOC_MAX_NODES = 1048576,
    VMHIP_NOALLOC_MAX_RANGES = 65536
};
typedef struct vmhip_projection_device {
    int32_t capacity;
    int32_t* n_visible;
    float* pixel_coordinates;
    int32_t* global_indices;
    int32_t* neighbourhood;
} vmhip_projection_device;
int vmhip_project_noalloc(const vmhip_mesh* mesh, const float* Rco, const vmhip_lens* lens, const int32_t* ranges,
                          int32_t n_ranges, int32_t n_candidates, const vmhip_projection_device* out, void* hip_stream);

/* What a consumer of the classified mesh does first, done on the device so that only detections cross PCIe. No
 * counterpart inside the reference's engines: its consumers walk the whole ClassifiedMesh on the host
 * (example/draw.hpp:41-59), over the neighbourhood table of engine/cpu/engine.hpp:113-129.
 * A node of a frame is detected if its probability of class_index is at least threshold and, with arg_max_only != 0,
 * no other class has a larger one (of equal ones the first wins, like std::max_element). Detections keep the order
 * of the visible nodes. With clusters != 0 they are also grouped into the connected components of the neighbourhood
 * graph restricted to the detections; clusters are numbered by their first detection.
 * Per frame: capacity / cluster_capacity say how much the caller's arrays hold; n_detections / n_clusters are
 * always written; if a capacity is too small the call returns VMHIP_ERR_CAPACITY and copies nothing.
 * Any array pointer may be NULL to skip that output. */
typedef struct vmhip_detections {
    int32_t capacity;
    int32_t cluster_capacity;
    int32_t n_detections;
    int32_t n_clusters;
    int32_t* node;         /* [n_detections] index into the mesh */
    float* pixel;          /* [n_detections][2] */
    float* probability;    /* [n_detections] */
    int32_t* cluster;      /* [n_detections] cluster number */
    int32_t* cluster_size; /* [n_clusters] */
    float* cluster_box;    /* [n_clusters][4] min x, min y, max x, max y */
    float* cluster_centre; /* [n_clusters][2] mean pixel (summed in no fixed order: last bits may vary) */
} vmhip_detections;
/* works on the results of the last vmhip_batch_run of a batch staged with classify != 0; out has one entry per frame */
int vmhip_batch_detect(vmhip_batch* batch, int32_t class_index, float threshold, int32_t arg_max_only, int32_t clusters,
                       vmhip_detections* out);

/* Per-kernel timing of vmhip_batch_run with HIP events on the stream the kernels run on.
 * enable = 1 brackets every kernel launch of later runs with events (such runs are launched kernel by kernel, and an
 * event pair between two kernels costs a few microseconds of idle GPU); enable = 2, valid after a run made with
 * enable = 1, brackets only the launches of the kernel that took longest in that run (such runs replay the batch's
 * captured graph like untimed ones, with the event records as nodes of it); 0 switches timing off.
 * After a run, vmhip_batch_profile_read returns, for kernel slot i < *n_slots, its name (static string), the
 * duration in milliseconds of its launch in the last run and the rows (nodes incl. null rows) or
 * candidates it processed. Slots are in launch order (with enable = 2: the bracketed launches only). */
int vmhip_batch_profile(vmhip_batch* batch, int32_t enable);
int vmhip_batch_profile_read(vmhip_batch* batch, int32_t max_slots, int32_t* n_slots, const char** names,
                             float* milliseconds, int64_t* units);

/* Test knobs, process wide, with no counterpart in the reference. They exist so that tests can drive paths that never
 * run on a healthy system, with every kernel still ending normally; production code has no use for them.
 *   VMHIP_DEBUG_FLOW_POLL_LIMIT   polls a wave of the barrier-free convolution kernel waits for a tile before it gives
 *                                 up and the run fails (takes effect at once; <= 0 restores the default)
 *   VMHIP_DEBUG_PROJECTION_ERROR  pixels added to both coordinates of every projected node on the device, as if the
 *                                 device's lens arithmetic differed from the host's: the host's re-decision of near-edge
 *                                 nodes must then overrule the device (read when a batch is staged; 0 = off)
 *   VMHIP_DEBUG_EDGE_BAND         width in pixels of the band along the screen edges inside which nodes are re-decided
 *                                 on the host (read when a batch is staged; <= 0 restores the default, 1/64)
 *   VMHIP_DEBUG_WIDE_OFFSETS      non-zero: the neighbourhood kernel addresses its tables with 64-bit offsets, as it does by
 *                                 itself for a batch with a table of 4 GiB or more (read when a batch is staged; 0 = off)
 *   VMHIP_DEBUG_STAMP_ROW_BITS    24..31: the entries of the reverse lookup keep at least that many bits for the row, as
 *                                 they do by themselves for a frame of 2^24 candidates or more, and so fewer for the run
 *                                 stamp: the table is then cleared every 2^(32 - bits) - 1 runs (read when a batch is
 *                                 staged; 0 = off) */
enum {
    VMHIP_DEBUG_FLOW_POLL_LIMIT = 0,
    VMHIP_DEBUG_PROJECTION_ERROR = 1,
    VMHIP_DEBUG_EDGE_BAND = 2,
    VMHIP_DEBUG_WIDE_OFFSETS = 3,
    VMHIP_DEBUG_STAMP_ROW_BITS = 4
};
int vmhip_debug_set(int32_t what, double value);
/* What the edge guard did in the runs of a batch since it was staged: near-edge nodes the device listed (summed over
 * frames and passes), the most it listed for one frame in one pass, device decisions the host overruled, passes
 * repeated because of that. The last two are zero on a host whose C library is the one the device arithmetic
 * reproduces. Any pointer may be NULL. */
int vmhip_batch_guard_stats(const vmhip_batch* batch, int64_t* listed, int64_t* most_listed, int64_t* overruled, int64_t* reruns);

/* Diagnostic with no counterpart in the reference: evaluates on the device, for n floats, the library's
 * own acosf (which = 0), sinf (1), tanf (2) or sqrtf (3) - the functions the lens projection is built from
 * and which must return the host C library's bits. x and y are host buffers. */
int vmhip_selftest_libm(int32_t which, const float* x, float* y, int32_t n);
/* Diagnostic with no counterpart in the reference: runs a plain device-to-device copy kernel of `bytes`
 * bytes (a multiple of 16) `repeats` times and returns the average milliseconds per launch in *ms. Profilers
 * use it as the dispatch of known size that hardware memory counters are scaled by; it also gives the
 * practical copy bandwidth of the device. */
int vmhip_selftest_copy(int64_t bytes, int32_t repeats, float* ms);
/* Diagnostic with no counterpart in the reference: a graph-convolution layer reduced to its memory traffic - `rows` rows
 * (a multiple of 64), `read_bytes_per_row` read and `write_bytes_per_row` written (multiples of 4), whole cache lines,
 * no arithmetic - run `repeats` times; the average milliseconds per launch go to *ms. What it reaches is what the memory
 * system gives a kernel with that mix of reads and writes at best: the ceiling the gather-bound layers are measured
 * against next to the 8 TB/s peak. */
int vmhip_selftest_stream(int64_t rows, int32_t read_bytes_per_row, int32_t write_bytes_per_row, int32_t repeats, float* ms);

/* ---- Scalar = double ----
 * The reference's engines and meshes are templates over Scalar (engine/cpu/engine.hpp:49-50, mesh.hpp:56; the training
 * op registers float and double, tensorflow/lookup.cpp:255-278). These entry points are what Engine<double> binds: the
 * same path as vmhip_project / vmhip_classify with every stage in fp64 on the device - projection, the strict on-screen
 * filter, compaction, the neighbourhood table, sampling, and the layers on the fp64 matrix cores. The mesh must be the
 * one Mesh<double, Model> generates (a double mesh is not the float mesh rounded: ring sizes come from ceil() of
 * quotients in Scalar), the ranges what its lookup returns. One frame per call; structures and meanings mirror the float
 * ones above. Layers may have any number of inputs; a softmax layer at most 128 outputs. */
typedef struct vmhip_lens_f64 {
    int32_t width, height;
    int32_t projection;
    double focal_length;
    double centre[2];
    double k[2];
    double fov;
} vmhip_lens_f64;
typedef struct vmhip_layer_f64 {
    int32_t n_in, n_out;
    int32_t activation;
    const double* weights; /* [n_in][n_out] row major */
    const double* biases;  /* [n_out] */
} vmhip_layer_f64;
typedef struct vmhip_network_f64 {
    int32_t n_groups;
    const int32_t* group_sizes;
    const vmhip_layer_f64* layers;
} vmhip_network_f64;
typedef struct vmhip_engine_f64 vmhip_engine_f64;
typedef struct vmhip_mesh_f64 vmhip_mesh_f64;
typedef struct vmhip_frame_f64 {
    const vmhip_mesh_f64* mesh;
    double Rco[9];         /* row major; Rco[i][j] = Hoc[j][i] */
    vmhip_lens_f64 lens;
    const int32_t* ranges; /* n_ranges pairs (first, one-past-last), ascending and disjoint */
    int32_t n_ranges;
    const void* image;     /* NULL when only projecting */
    uint32_t fourcc;
} vmhip_frame_f64;
typedef struct vmhip_result_f64 {
    int32_t capacity;  /* in nodes: at least the sum of the range lengths */
    int32_t n_visible; /* written by the library */
    double* pixel_coordinates; /* [capacity][2] */
    int32_t* global_indices;   /* [capacity] */
    int32_t* neighbourhood;    /* [capacity+1][n_neighbours] */
    double* classifications;   /* [capacity+1][n_classes]; may be NULL when projecting */
} vmhip_result_f64;
/* Replaces cpu::Engine<double>'s constructor (reference engine/cpu/engine.hpp:57-71). */
int vmhip_engine_create_f64(const vmhip_network_f64* net, int32_t n_neighbours, vmhip_engine_f64** out);
void vmhip_engine_destroy_f64(vmhip_engine_f64* engine);
int32_t vmhip_engine_n_classes_f64(const vmhip_engine_f64* engine);
/* rays[n_nodes][3] of doubles, neighbours[n_nodes][n_neighbours] as for vmhip_mesh_upload */
int vmhip_mesh_upload_f64(const double* rays, const int32_t* neighbours, int32_t n_nodes, int32_t n_neighbours,
                          vmhip_mesh_f64** out);
void vmhip_mesh_release_f64(vmhip_mesh_f64* mesh);
/* Replace cpu::Engine<double>::operator()(mesh, Hoc, lens) and (mesh, Hoc, lens, image, format)
 * (reference engine/cpu/engine.hpp:84-147, :180-273). */
int vmhip_project_f64(vmhip_engine_f64* engine, const vmhip_frame_f64* frame, vmhip_result_f64* result);
int vmhip_classify_f64(vmhip_engine_f64* engine, const vmhip_frame_f64* frame, vmhip_result_f64* result);
/* What the edge guard of a double engine did since the engine was made (see vmhip_batch_guard_stats): near-edge nodes
 * the device listed, device decisions the host overruled. Either pointer may be NULL. */
int vmhip_engine_guard_stats_f64(const vmhip_engine_f64* engine, int64_t* listed, int64_t* overruled);

#ifdef __cplusplus
}
#endif
#endif

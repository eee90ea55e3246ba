/*
 * Internal definitions shared by the kernels and the C ABI implementation of libvisualmesh_hip.so.
 *
 * Device memory layout of a staged batch
 * --------------------------------------
 * Two index spaces, both tiled by TILE (256) and laid out frame after frame:
 *   candidate space: one slot per node in the frame's lookup ranges (slot p of frame f lives at
 *                    cand_base[f] + p). Holds the projected pixel and the keep mask.
 *   row space:       one row per visible node plus the null row (row i of frame f lives at
 *                    row_base[f] + i). Capacity per frame = candidates + 1 rounded up to TILE, because
 *                    the visible count is only known on the device. Holds pixel coordinates, global
 *                    indices, the neighbourhood table and the ping/pong activation matrices.
 * A tile never straddles two frames, so every block works for exactly one frame and finds it by a
 * binary search over the frames' first-tile numbers.
 *
 * Tile-local gather tables (built once per run next to the neighbourhood table, used by every layer):
 * mesh order is spatially coherent, so most of a row's neighbours live in the row's own tile and the rest
 * of a tile's neighbours are ~100 distinct rows of other tiles (its halo). tile_halo lists those rows,
 * row_nbl holds every neighbour as a position in "the tile's 256 rows followed by its halo rows", and
 * tile_desc describes the tile in one 16-byte word. A layer kernel copies tile + halo rows into LDS with
 * coalesced loads and gathers from there.
 */
#ifndef VMHIP_INTERNAL_H
#define VMHIP_INTERNAL_H

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "visualmesh_hip.h"

#define VMHIP_TILE 256
#define VMHIP_AMB_CAP 2048 /* ambiguous candidates recorded per frame */
#define VMHIP_HALO_MAX 256 /* rows of other tiles that a row tile can stage next to its own 256 rows */
#define VMHIP_NBL_STRIDE 8 /* tile-local neighbour table: 8 x uint16 per row */
#define VMHIP_NBL_FAR 0xffffu /* tile-local neighbour entry: not staged, read the row from global memory */
/* the bf16 layers (conv_bf16.hip) work on half tiles: 128 rows and up to 128 rows of other half tiles, so that two
 * buffers of 256-byte rows fit the LDS beside each other */
#define VMHIP_HTILE 128
#define VMHIP_HHALO 128
#define VMHIP_NOTE_WORDS (4 + VMHIP_HHALO) /* a half tile's note: {first row, rows in use, halo rows, frame's first row}, then its halo rows */

/* how the rows of an activation matrix are stored (VmLayerDev::in_bf16 / out_bf16) */
enum {
    VM_ROWS_F32 = 0,    /* C floats */
    VM_ROWS_BF16 = 1,   /* C bf16: the value rounded once */
    VM_ROWS_BF16X2 = 2  /* C bf16 "hi" then C bf16 "lo", hi = bf16(x), lo = bf16(x - hi): 16 significant bits, ready as matrix operands */
};

/* image sampling kinds (derived from the fourcc on the host) */
enum {
    VMHIP_FMT_RGBA = 0,
    VMHIP_FMT_BGRA = 1,
    VMHIP_FMT_RGB3 = 2,
    VMHIP_FMT_BGR3 = 3,
    VMHIP_FMT_GRAY = 4,
    VMHIP_FMT_GRBG = 5,
    VMHIP_FMT_RGGB = 6,
    VMHIP_FMT_GBRG = 7,
    VMHIP_FMT_BGGR = 8,
    VMHIP_FMT_NONE = 9
};

struct VmFrame {
    /* mesh */
    const float* rays;     /* [n_nodes][3] */
    const int32_t* nbr;    /* [n_nodes][nn] */
    uint32_t* r_lookup;    /* [n_nodes+1] run stamp above the local row (VmBatchDev::stamp_row_bits); entry n_nodes is never stamped */
    int32_t n_nodes;
    int32_t nn;
    /* pose + lens */
    float Rco[9];
    float focal, centre_x, centre_y;
    float ik[4];           /* inverse distortion coefficients, computed on the host in fp32 */
    int32_t width, height, projection;
    /* image */
    const uint8_t* image;
    int32_t fmt;
    /* lookup ranges */
    const int32_t* range_first;  /* [n_ranges] first global index of each range */
    const int32_t* range_prefix; /* [n_ranges+1] exclusive prefix sum of range lengths */
    int32_t n_ranges;
    int32_t n_cand;
    /* placement */
    int32_t cand_base, cand_tile0, cand_tiles;
    int32_t row_base, row_tile0, row_tiles;
    /* forced decisions for candidates the host re-decided: bit set in force_valid -> take force_keep */
    const uint64_t* force_valid; /* indexed like the keep mask: (cand_base + p) / 64 */
    const uint64_t* force_keep;
};

/* What changes from one staged batch to the next while every address and launch grid stays the same: the tiles in use.
 * It lives in device memory (uploaded with the frame descriptions), so that a pass captured into a HIP graph with one
 * batch serves the batches staged after it. */
struct VmBatchLive {
    int32_t n_cand_tiles, n_row_tiles;
};

struct VmBatchDev {
    const VmFrame* frames;
    int32_t n_frames;
    /* the tiles the launch grids are sized for: at least the tiles in use, which kernels read through `live` */
    int32_t n_cand_tiles, n_row_tiles;
    const VmBatchLive* live; /* null: the two counts above are the tiles in use */
    uint32_t* epoch;      /* device word: the run's stamp for the reverse lookup, from 1; the last kernel of a pass increments it */
    /* where a tile belongs, worked out when the batch is staged so that no block has to search for it (null: the blocks search) */
    const int2* cand_tile_info;     /* [n_cand_tiles] {frame, index of the range that holds the tile's first candidate} */
    const int32_t* row_tile_frame;  /* [n_row_tiles] frame */
    int32_t uniform_nn;     /* neighbours per node if every frame of the batch has the same number, else 0 */
    int32_t wide_offsets;   /* a frame's part of a table reaches 4 GiB: the neighbourhood kernel addresses with 64-bit offsets */
    int32_t stamp_row_bits; /* a reverse-lookup entry is (stamp << stamp_row_bits) | local row: 24 bits of row unless a frame
                             * has 2^24 candidates or more; the stamp counts from 1 to 2^(32 - stamp_row_bits) - 1 and the table
                             * is cleared before it starts again */
    /* candidate space */
    float2* cand_px;
    int32_t* cand_g;      /* the candidate's node (global index), worked out once by the projection */
    uint64_t* cand_keep;  /* one 64-bit mask per wave of candidates */
    int32_t* tile_count;  /* [n_cand_tiles] kept candidates per tile */
    /* per frame */
    int32_t* frame_V;     /* [n_frames] visible nodes */
    int32_t* amb_count;   /* [n_frames] */
    int2* amb_list;       /* [n_frames][VMHIP_AMB_CAP] {candidate slot, gpu decision} */
    /* row space */
    float2* row_px;
    int32_t* row_gidx;
    int32_t* row_nb;      /* [rows][nn_max] with the frame's own nn as stride */
    int32_t nb_stride;
    /* tile-local gather tables (null unless the batch classifies and nn <= VMHIP_NBL_STRIDE) */
    uint16_t* row_nbl;    /* [rows][VMHIP_NBL_STRIDE]: 0..255 own tile, 256+h halo slot h, VMHIP_NBL_FAR not staged */
    uint32_t* tile_halo;  /* [n_row_tiles][VMHIP_HALO_MAX] batch-global row of each halo slot */
    int4* tile_desc;      /* [n_row_tiles] {first batch-global row, rows in use (0..256), halo rows, frame's row_base} */
    int32_t halo_cap;     /* halo slots handed out per tile, <= VMHIP_HALO_MAX (smaller only to test the far path) */
    /* the same for half tiles (null unless the engine has bf16 layers). Only half tiles with rows in use are numbered:
     * half tile t of frame f is number active_h[f] + t */
    int32_t* active_h;    /* [n_frames + 1] half tiles in use before each frame; the last entry is their total */
    uint16_t* row_nbl_h;  /* [rows][VMHIP_NBL_STRIDE]: 0..127 own half tile, 128+h halo slot h, VMHIP_NBL_FAR not staged */
    uint32_t* tile_note_h; /* [half tiles in use][VMHIP_NOTE_WORDS] */
    unsigned int* flow_timeouts; /* the batch's count of waits of the barrier-free kernel that ran out of polls (0 in a correct run) */
    /* edge guard: a candidate closer than amb_eps pixels to a screen edge is listed for the host's re-decision.
     * px_error is 0 outside tests: added to both pixel coordinates, it stands for a device whose lens arithmetic
     * differs from the host's (vmhip_debug_set) */
    float amb_eps, px_error;
};
/* the tiles in use, on the device (uniform: scalar loads) */
__device__ __forceinline__ int vm_cand_tiles(const VmBatchDev& B) { return B.live ? B.live->n_cand_tiles : B.n_cand_tiles; }
__device__ __forceinline__ int vm_row_tiles(const VmBatchDev& B) { return B.live ? B.live->n_row_tiles : B.n_row_tiles; }
#define VMHIP_AMB_EPS_DEFAULT 0.015625f /* 1/64 px: far above any device/host libm difference, far below node spacing */

/* Lookup on the device (project.hip: vm_lookup_kernel): the cone tree over a mesh's nodes and what a frame's walk of it
 * needs. The tree, the walk and every comparison in it are those of the host's lookup (cpp/visualmesh/detail/
 * cone_tree.hpp), so the ranges are the same. */
struct VmTreeElement {
    int32_t first, last; /* node range [first, last) */
    int32_t child[2];    /* -1, -1 for a leaf */
    float axis[3], c, s; /* bounding cone: axis, cosine and sine of its half angle */
};
struct VmLookupFrame {
    VmFrame frame;              /* rays, n_nodes, pose, lens: what project_ray reads */
    const VmTreeElement* tree;
    int32_t n_elements;
    float cos_half_fov, sin_half_fov;
    float edge[4][5];           /* the four screen-edge cones: axis, cosine, sine */
    uint32_t* covered;          /* [ceil(n_nodes / 32)] one bit per node */
    int32_t* list[2];           /* [n_elements] each: the walk's frontiers, then the runs' starts and ends */
    int32_t capacity;           /* ranges a frame may produce: n_elements */
    int32_t* cursor;            /* one word for the whole launch: next free word of `dense` */
    int32_t* dense;             /* every frame's first[n] and prefix[n + 1], one frame after the other */
    int32_t* verdict;           /* [3] ranges (-1: more than capacity), candidates, offset into dense */
};
void vm_launch_lookup(const VmLookupFrame* frames, int n_frames, hipStream_t stream);
/* vectors [cand][3], pixels [cand][2] at the frames' candidate bases; graph rows of nn+1 words, a frame's block at
 * cand_base * (nb_stride + 1) */
void vm_launch_lookup_export(const VmBatchDev& B, int same_edges, float* vectors, int32_t* graph, float* pixels, hipStream_t stream);

/* Layer descriptor on the device side (host struct, passed by value to launchers). */
struct VmLayerDev {
    int32_t c_in;    /* width of one gathered row */
    int32_t c_out;
    int32_t slots;   /* nn+1 for the first layer of a group, 1 for the dense layers after it */
    int32_t activation;
    const float* w;  /* [slots*c_in][c_out] fp32 row major */
    const float* b;  /* [c_out] */
    const void* w_mfma; /* the same weights in the matrix-core kernel's consumption order, or null */
    int32_t in_bf16;    /* how the input rows are stored: VM_ROWS_* */
    int32_t out_bf16;   /* how the output rows are stored: VM_ROWS_* */
    int32_t arith_bf16; /* bf16 products with fp32 accumulation (weights in w_mfma are bf16 then) */
    const float* w_flow; /* the fp32 w_mfma weights in the order conv_flow.hip keeps them in LDS, or null */
};

/* Device side of the detection step (detect.hip): every array is indexed like the row space, a frame's entries
 * starting at its row_base, so the worst case (every node detected, every detection its own cluster) fits. */
struct VmDetectDev {
    const float* probabilities; /* the last run's final activations, [rows][n_classes] */
    int32_t n_classes, class_index, arg_max_only;
    float threshold;
    int32_t* node;             /* mesh index of each detection */
    float2* pixel;
    float* probability;
    int32_t* cluster;          /* cluster number of each detection */
    int32_t* row_to_detection; /* per row: its detection number or -1 */
    int32_t* parent;           /* union-find over a frame's detections */
    int32_t* cluster_size;
    int32_t* cluster_box;      /* [4] min x, min y, max x, max y as float bits */
    float* cluster_sum;        /* [2] sum of pixels */
    int32_t* counts;           /* [n_frames][2] detections, clusters */
};
#define VM_DETECT_BYTES_PER_ROW 64 /* 56 used, the rest covers the 16-byte alignment of each array */
size_t vm_detect_workspace_bytes(size_t rows, int n_frames);
/* points D's arrays into a workspace of that size (counts last, n_frames * 8 bytes) */
void vm_detect_carve(void* workspace, size_t rows, int n_frames, VmDetectDev* D);
void vm_launch_detect(const VmBatchDev& B, const VmDetectDev& D, int clusters, hipStream_t stream);
/* packed: 5 * total_d + 7 * total_c words (detect.hip says in which order) */
void vm_launch_detect_pack(const VmBatchDev& B, const VmDetectDev& D, uint32_t* packed, int total_d, int total_c, hipStream_t stream);
/* one array of one frame on its way into the block of vmhip_batch_fetch_packed_async (detect.hip: vm_fetch_pack_kernel) */
#define VM_PACK_CHUNK 16384
struct VmPackSegment {
    const uint8_t* src;
    size_t dst_offset, bytes;        /* multiples of 256 and of 4 */
    size_t row_bytes, src_stride;    /* equal for a contiguous array */
    int32_t chunk_first;             /* number of the segment's first chunk of VM_PACK_CHUNK bytes */
};
void vm_launch_fetch_pack(const VmPackSegment* segments, int n_segments, int n_chunks, void* dst, hipStream_t stream);

/* "<family>_<c_in>x<c_out>s<slots>" as a string that stays valid (the profile of a run names its kernels) */
const char* vm_kernel_name(const char* family, int c_in, int c_out, int slots);

/* launchers, one per kernel; all asynchronous on `stream` */
void vm_launch_libm(int which, const float* x, float* y, int n, hipStream_t stream);
void vm_launch_copy_probe(const void* src, void* dst, size_t bytes, hipStream_t stream);
/* rows: a multiple of 64; bytes per row: multiples of 4 (64 rows are whole 16-byte pieces then) */
void vm_launch_stream_probe(const void* src, void* dst, size_t rows, int read_bytes_per_row, int write_bytes_per_row, hipStream_t stream);
/* counts[n_counts], the first amb_head entries of every frame's ambiguity list and the timeout count, stored by the device
 * into page-locked host memory (device-visible pointers) */
void vm_launch_publish(int32_t* counts, int n_counts, const int2* amb_list, int amb_stride, int amb_head, int n_frames, const unsigned int* timeouts, uint32_t* epoch,
                       int32_t* host_counts, int2* host_amb, uint32_t* host_timeouts, hipStream_t stream);
void vm_launch_project(const VmBatchDev& B, hipStream_t stream);
void vm_launch_compact(const VmBatchDev& B, float* feat, int classify, hipStream_t stream);
void vm_launch_neighbourhood(const VmBatchDev& B, hipStream_t stream); /* also the tile-local tables if B.row_nbl */
/* the same launch with the network's first layer (4 sampled channels in, up to 32 out) computed by the blocks for their
 * own tiles: `in` = the sampled rows, `out` = the layer's rows; a negative value if the layer or the batch does not fit
 * (then nothing was launched) */
bool vm_neighbourhood_conv_supported(int c_in, int c_out, int slots, int activation);
int vm_launch_neighbourhood_conv(const VmBatchDev& B, const VmLayerDev& L, const float* in, float* out, hipStream_t stream, const char** kernel_name);
/* in -> out over the row space; returns 0 or a negative status if the shape is unsupported */
int vm_launch_conv(const VmBatchDev& B, const VmLayerDev& L, const float* in, float* out, hipStream_t stream,
                   const char** kernel_name);

/* matrix-core variant (conv_mfma.hip); launch returns a negative value if the combination has no instantiation */
bool vm_mfma_supported(int c_in, int c_out, int slots);
size_t vm_mfma_weight_bytes(int c_in, int c_out, int slots);
void vm_mfma_permute_weights(const float* w, int c_in, int c_out, int slots, void* wp);
int vm_launch_conv_mfma(const VmBatchDev& B, const VmLayerDev& L, const void* in, void* out, hipStream_t stream,
                        const char** kernel_name);

/* the bf16 engine's layers (conv_bf16.hip): bf16 matrix instructions with fp32 accumulation, weights in registers, rows
 * of half tiles staged in LDS. vm_launch_half_tables builds the half-tile tables from the neighbour table of the run. */
bool vm_bf16_supported(int c_in, int c_out, int slots);
size_t vm_bf16_weight_bytes(int c_in, int c_out, int slots);
void vm_bf16_permute_weights(const float* w, int c_in, int c_out, int slots, int out_fmt, void* wp);
void vm_launch_half_tables(const VmBatchDev& B, hipStream_t stream);
int vm_launch_conv_bf16(const VmBatchDev& B, const VmLayerDev& L, const void* in, void* out, hipStream_t stream,
                        const char** kernel_name);

/* matrix-core variant gathering from LDS through the tile-local tables (conv_lds.hip); fp32 rows and arithmetic,
 * weights in vm_mfma_permute_weights' fp32 order; writes fp32 rows, or hi + lo rows for a bf16 layer to read */
bool vm_lds_supported(int c_in, int c_out, int slots, int out_fmt = VM_ROWS_F32);
int vm_launch_conv_lds(const VmBatchDev& B, const VmLayerDev& L, const float* in, float* out, hipStream_t stream,
                       const char** kernel_name);

/* A row of the tile-local neighbour table, read with a load exactly as wide as the NN entries in use. A wider load
 * leaves dead result registers; the compiler reuses them at once, and that reuse must wait for the load - and for every
 * load issued before it - to return. */
template <int NN>
__device__ __forceinline__ __attribute__((ext_vector_type(4))) uint32_t vm_load_nbl_row(__amdgpu_buffer_rsrc_t rsrc, int byte_offset) {
    typedef uint32_t u2 __attribute__((ext_vector_type(2)));
    typedef uint32_t u3 __attribute__((ext_vector_type(3)));
    typedef uint32_t u4 __attribute__((ext_vector_type(4)));
    if constexpr (NN <= 2) {
        return u4{__builtin_amdgcn_raw_buffer_load_b32(rsrc, byte_offset, 0, 0), 0u, 0u, 0u};
    }
    else if constexpr (NN <= 4) {
        const u2 t = __builtin_amdgcn_raw_buffer_load_b64(rsrc, byte_offset, 0, 0);
        return u4{t.x, t.y, 0u, 0u};
    }
    else if constexpr (NN <= 6) {
        const u3 t = __builtin_amdgcn_raw_buffer_load_b96(rsrc, byte_offset, 0, 0);
        return u4{t.x, t.y, t.z, 0u};
    }
    else {
        return __builtin_amdgcn_raw_buffer_load_b128(rsrc, byte_offset, 0, 0);
    }
}

/* the same with rows brought into LDS by buffer_load ... lds, two alternating row buffers and LDS counters in place of the tile loop's barriers, so that the waves of a block run freely between
 * "my tile is staged" and "my buffer may be refilled" (conv_flow.hip) */
bool vm_flow_supported(int c_in, int c_out, int slots);
/* host side: w_mfma (fp32, vm_mfma_permute_weights' order) rearranged into that kernel's LDS order; same size */
void vm_flow_order_weights(const float* w_mfma, int c_in, int c_out, int slots, float* out);
int vm_launch_conv_flow(const VmBatchDev& B, const VmLayerDev& L, const float* in, float* out, hipStream_t stream,
                        const char** kernel_name);
#define VM_FLOW_POLL_LIMIT_DEFAULT (1 << 22)
hipError_t vm_flow_set_poll_limit(int polls); /* process wide; tests of the give-up path only */

/* layers with at most four output channels on v_mfma_f32_4x4x1 (64 rows x 4 channels per instruction), staged like
 * conv_flow.hip (conv_narrow.hip); reads the plain row-major weights */
bool vm_narrow_supported(int c_in, int c_out, int slots);
int vm_launch_conv_narrow(const VmBatchDev& B, const VmLayerDev& L, const float* in, float* out, hipStream_t stream,
                          const char** kernel_name);

#include "host_project.h"

#include <vector>

/* a mesh on the device (api.hip: vmhip_mesh_upload) */
struct vmhip_mesh {
    float* d_rays = nullptr;
    int32_t* d_nbr = nullptr;
    int32_t n_nodes = 0, nn = 0;
    int device = 0;            /* the device that holds it */
    std::vector<float> h_rays; /* host copy for the re-decision of ambiguous candidates */
    VmTreeElement* d_tree = nullptr; /* the cone tree, for lookups on the device (vmhip_mesh_attach_tree) */
    int32_t n_elements = 0;
};

/* noalloc.hip: the entry point that allocates nothing. vm_noalloc_setup finds the current device's copy of that file's
 * scratch array (once per device; mesh uploads call it, so the entry point itself finds it done); vm_set_error records
 * the calling thread's message for vmhip_last_error and returns code. */
hipError_t vm_noalloc_setup(void);
int vm_set_error(int code, const char* message);
/* fourcc -> sampling kind (VMHIP_FMT_*) and bytes per pixel; false for a code the reference's pixel.hpp does not take */
bool vm_decode_fourcc(uint32_t fourcc, int* fmt, int* bytes_per_pixel);
/* the test knobs VMHIP_DEBUG_PROJECTION_ERROR and VMHIP_DEBUG_EDGE_BAND as they stand */
void vm_debug_knobs(double* projection_error, double* edge_band);

#endif

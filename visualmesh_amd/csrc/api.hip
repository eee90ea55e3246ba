/*
 * api.hip - the C ABI of libvisualmesh_hip.so (include/visualmesh_hip.h): engine, mesh and batch objects,
 * staging, the launch sequence, the host re-decision of edge-ambiguous candidates, result download.
 */
#include <algorithm>
#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <string>
#include <vector>

#include "visualmesh_hip.h"
#include "vmhip_internal.h"

namespace {

thread_local std::string g_error;

/* test knobs (vmhip_debug_set); read when a batch is staged */
std::atomic<float> g_debug_px_error{0.0f};
std::atomic<bool> g_debug_wide_offsets{false};
std::atomic<int> g_debug_stamp_row_bits{0};
std::atomic<float> g_debug_edge_band{VMHIP_AMB_EPS_DEFAULT};
std::atomic<int> g_live_engines{0}; /* engines alive in the process, each with a stream of its own */

int fail(int code, const std::string& msg) {
    g_error = msg;
    return code;
}
#define HIP_TRY(expr)                                                                                  \
    do {                                                                                               \
        hipError_t e_ = (expr);                                                                        \
        if (e_ != hipSuccess)                                                                          \
            return fail(VMHIP_ERR_HIP, std::string(#expr) + " failed: " + hipGetErrorString(e_));      \
    } while (0)

/* grow-only device allocation */
struct DevBuf {
    void* p = nullptr;
    size_t cap = 0;
    bool grew = false;
    hipError_t reserve(size_t bytes) {
        grew = false;
        if (bytes <= cap) return hipSuccess;
        if (p) {
            hipError_t e = hipFree(p);
            p = nullptr;
            cap = 0;
            if (e != hipSuccess) return e;
        }
        const size_t want = bytes + bytes / 8 + 256;
        hipError_t e = hipMalloc(&p, want);
        if (e != hipSuccess) {
            p = nullptr;
            return e;
        }
        cap = want;
        grew = true;
        return hipSuccess;
    }
    void release() {
        if (p) (void) hipFree(p);
        p = nullptr;
        cap = 0;
    }
    template <typename T>
    T* as() const {
        return reinterpret_cast<T*>(p);
    }
};

inline uint32_t cc(char a, char b, char c, char d) {
    return uint32_t(uint8_t(a)) | (uint32_t(uint8_t(b)) << 8) | (uint32_t(uint8_t(c)) << 16) | (uint32_t(uint8_t(d)) << 24);
}
/* fourcc -> sampling kind and bytes per pixel; the accepted codes are those of reference
 * engine/cpu/pixel.hpp:48-97 */
bool decode_fourcc(uint32_t f, int* fmt, int* bpp) {
    if (f == cc('R', 'G', 'B', 'A')) return *fmt = VMHIP_FMT_RGBA, *bpp = 4, true;
    if (f == cc('B', 'G', 'R', 'A')) return *fmt = VMHIP_FMT_BGRA, *bpp = 4, true;
    if (f == cc('R', 'G', 'B', '3') || f == cc('R', 'G', 'B', '8')) return *fmt = VMHIP_FMT_RGB3, *bpp = 3, true;
    if (f == cc('B', 'G', 'R', '3') || f == cc('B', 'G', 'R', '8')) return *fmt = VMHIP_FMT_BGR3, *bpp = 3, true;
    if (f == cc('G', 'R', 'A', 'Y') || f == cc('G', 'R', 'E', 'Y') || f == cc('Y', '8', ' ', ' '))
        return *fmt = VMHIP_FMT_GRAY, *bpp = 1, true;
    if (f == cc('G', 'R', 'B', 'G')) return *fmt = VMHIP_FMT_GRBG, *bpp = 1, true;
    if (f == cc('R', 'G', 'G', 'B')) return *fmt = VMHIP_FMT_RGGB, *bpp = 1, true;
    if (f == cc('G', 'B', 'R', 'G')) return *fmt = VMHIP_FMT_GBRG, *bpp = 1, true;
    if (f == cc('B', 'G', 'G', 'R')) return *fmt = VMHIP_FMT_BGGR, *bpp = 1, true;
    return false;
}
std::string fourcc_text(uint32_t f) {
    char t[5] = {char(f & 0xff), char((f >> 8) & 0xff), char((f >> 16) & 0xff), char((f >> 24) & 0xff), 0};
    return std::string(t);
}

inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

}  // namespace

struct HostLayer {
    int32_t c_in, c_out, slots, activation;
    float* d_w = nullptr;
    float* d_b = nullptr;
    void* d_w_mfma = nullptr;
    float* d_w_flow = nullptr; /* w_mfma in conv_flow.hip's LDS order */
    int32_t in_bf16 = 0, out_bf16 = 0, arith_bf16 = 0;
    bool use_lds = false, use_mfma = false, use_flow = false, use_narrow = false; /* which matrix-core kernels may take the layer */
    bool fuse_first = false; /* the network's first layer, computed by the neighbourhood kernel's blocks for their own tiles */
    std::vector<float> h_w, h_b; /* kept until the row types are planned */
};

struct vmhip_engine {
    bool use_graph = true;               /* VMHIP_GRAPH=0: launch every run kernel by kernel */
    bool use_lds = false;                /* some layer gathers through the tile-local tables */
    bool use_flow = false;               /* some layer runs the kernel that polls LDS counters instead of barriers */
    bool use_bf16 = false;               /* some layer runs on the bf16 matrix instructions (half-tile tables) */
    int32_t halo_cap = VMHIP_HALO_MAX;   /* VMHIP_HALO_CAP lowers it to exercise the not-staged path */
    int32_t nn = 0;
    int32_t precision = VMHIP_FP32;
    int32_t n_classes = 4;
    int32_t max_width = 4;
    std::vector<HostLayer> layers;
    hipStream_t stream = nullptr;
    bool counted = false;           /* in g_live_engines */
    vmhip_batch* scratch = nullptr; /* used by the one-call entry points */
};

struct HostFrame {
    const vmhip_mesh* mesh;
    std::vector<int32_t> first, prefix; /* host copies of the range table */
    VmFrame dev;
    float centre[2];
};

struct vmhip_batch {
    vmhip_engine* engine = nullptr;
    int32_t classify = 0;
    std::vector<HostFrame> frames;
    std::vector<int32_t> h_V, h_amb_count;
    std::vector<int2> h_amb;
    /* pinned landing area of the per-run download: V[n], ambiguity count[n], then the first AMB_HEAD entries of
     * every frame's ambiguity list, so that one wait per run covers everything the host normally needs */
    static constexpr int AMB_HEAD = 64;
    void* h_pin = nullptr;
    void* h_pin_dev = nullptr; /* the same memory as the device addresses it */
    size_t h_pin_cap = 0;
    std::vector<uint64_t> h_force_valid, h_force_keep;
    /* pinned home of the frame descriptions and range tables a stage uploads: they must outlive a stage that does not
     * wait for its copies */
    void* h_stage = nullptr;
    size_t h_stage_cap = 0;
    void* h_pack = nullptr; /* pinned home of the segment table of a packed fetch */
    size_t h_pack_cap = 0;
    bool stage_pending = false; /* copies of the last stage may still be reading h_stage (and the caller's images) */
    bool have_run = false;
    bool in_flight = false;     /* vmhip_batch_run_async without its vmhip_batch_wait */
    bool fetching = false;      /* vmhip_batch_fetch_async without its vmhip_batch_fetch_wait */
    uint64_t run_serial = 0;    /* counts completed runs */
    uint64_t detect_serial = 0; /* the run whose detections the workspace holds, with these parameters: */
    int32_t detect_class = -1, detect_arg_max = 0, detect_clusters = 0;
    float detect_threshold = 0.0f;
    uint32_t epoch = 0; /* host mirror of the device run stamp */
    int stamp_row_bits = 0; /* how the reverse-lookup entries of the table on the device are split (VmBatchDev::stamp_row_bits) */
    /* what the edge guard did since the batch was staged (vmhip_batch_guard_stats) */
    int64_t reruns = 0, overruled = 0, amb_seen = 0, amb_most = 0;
    /* The kernel sequence of a pass, captured into a HIP graph and replayed (VMHIP_GRAPH != 0, no per-kernel profiling).
     * What a captured pass holds is addresses, launch grids and the number of frames: the tiles in use, the frame
     * descriptions and every table are read from device memory, so the graph serves every batch staged after the one it
     * was captured with, until a buffer grows, a batch needs a larger grid or another number of frames, or the mode changes
     * (graph_key says what the capture was made with; batch_launch compares). */
    struct GraphKey {
        VmBatchDev dev;
        const void* act[2];
        const void* pin;
        int32_t classify, profile;
    };
    hipGraph_t graph = nullptr;
    hipGraphExec_t graph_exec = nullptr;
    GraphKey graph_key;
    int eager_runs = 0; /* passes launched kernel by kernel since the batch was made or its graph dropped: the first pass is
                         * launched that way (every kernel's one-time attribute set-up happens there), the second is captured */
    int64_t graph_captures = 0, graph_launches = 0, eager_launches = 0; /* vmhip_batch_graph_stats */
    void drop_graph() {
        if (graph_exec) (void) hipGraphExecDestroy(graph_exec);
        if (graph) (void) hipGraphDestroy(graph);
        graph_exec = nullptr, graph = nullptr, eager_runs = 0;
    }
    size_t cand_total = 0, row_total = 0, lookup_total = 0; /* slots the candidate and row spaces are allocated for */
    size_t cap_cand_tiles = 0, cap_row_tiles = 0;           /* the tiles the launch grids are sized for (>= the tiles in use) */
    VmBatchLive live{0, 0};                                  /* the tiles in use */
    /* the batch as the kernels outside the captured pass see it: grids of exactly the tiles in use */
    VmBatchDev dev_exact() const {
        VmBatchDev d = dev;
        d.n_cand_tiles = live.n_cand_tiles, d.n_row_tiles = live.n_row_tiles;
        return d;
    }

    VmBatchDev dev{};
    DevBuf d_frames, d_ranges, d_images, d_cand_px, d_cand_g, d_cand_keep, d_tile_count, d_force_valid, d_force_keep, d_frame_V,
      d_amb_list, d_row_px, d_row_gidx, d_row_nb, d_row_nbl, d_tile_halo, d_tile_desc, d_row_nbl_h, d_tile_note_h, d_active_h, d_act[2], d_lookup, d_epoch, d_detect, d_detect_packed, d_lookup_ws, d_export, d_fetch_packed;
    std::vector<std::vector<int32_t>> device_ranges; /* per frame: the ranges a lookup on the device produced */
    void* h_detect = nullptr; /* pinned landing area of vmhip_batch_detect */
    size_t h_detect_cap = 0;
    float* final_act = nullptr;

    /* profiling */
    int profile = 0; /* 0 off, 1 every kernel, 2 only the launches of the kernel that took longest in the last mode-1 run */
    std::vector<char> slot_wanted; /* mode 2: which launch slots are bracketed */
    std::vector<hipEvent_t> events;
    std::vector<const char*> slot_names;
    std::vector<int64_t> slot_units;
    int n_slots = 0;

    void release() {
        DevBuf* all[] = {&d_frames, &d_ranges, &d_images, &d_cand_px, &d_cand_g, &d_cand_keep, &d_tile_count, &d_force_valid,
                         &d_force_keep, &d_frame_V, &d_amb_list, &d_row_px, &d_row_gidx, &d_row_nb,
                         &d_row_nbl, &d_tile_halo, &d_tile_desc, &d_row_nbl_h, &d_tile_note_h, &d_active_h, &d_epoch,
                         &d_act[0], &d_act[1], &d_lookup, &d_detect, &d_detect_packed, &d_lookup_ws, &d_export, &d_fetch_packed};
        drop_graph();
        for (DevBuf* b : all) b->release();
        if (h_pin) (void) hipHostFree(h_pin);
        h_pin = nullptr, h_pin_cap = 0;
        if (h_stage) (void) hipHostFree(h_stage);
        h_stage = nullptr, h_stage_cap = 0;
        if (h_pack) (void) hipHostFree(h_pack);
        h_pack = nullptr, h_pack_cap = 0;
        if (h_detect) (void) hipHostFree(h_detect);
        h_detect = nullptr, h_detect_cap = 0;
        for (hipEvent_t e : events) (void) hipEventDestroy(e);
        events.clear();
    }
};

namespace {

int batch_stage(vmhip_batch* b, const vmhip_frame* frames, int32_t n_frames, int32_t classify, bool wait) {
    vmhip_engine* E = b->engine;
    if (!frames || n_frames <= 0) return fail(VMHIP_ERR_ARGUMENT, "stage: no frames");
    if (b->stage_pending) { /* staged twice without a run between: the first stage's copies still read h_stage */
        HIP_TRY(hipStreamSynchronize(E->stream));
        b->stage_pending = false;
    }
    b->have_run = false;
    b->classify = classify ? 1 : 0;
    b->frames.assign(n_frames, HostFrame());

    /* validate and place */
    size_t cand_tiles = 0, row_tiles = 0, range_ints = 0, image_bytes = 0, lookup_entries = 0, max_cand = 0;
    uint64_t widest_mesh = 0; /* most neighbour table entries of a frame's mesh */
    int32_t nb_stride = 1, uniform_nn = 0;
    for (int f = 0; f < n_frames; ++f) {
        const vmhip_frame& in = frames[f];
        HostFrame& hf = b->frames[f];
        if (!in.mesh) return fail(VMHIP_ERR_ARGUMENT, "stage: frame without a mesh");
        if (in.lens.projection < VMHIP_RECTILINEAR || in.lens.projection > VMHIP_EQUIDISTANT)
            return fail(VMHIP_ERR_LENS, "Cannot project: Unknown lens type");
        if (in.lens.width <= 0 || in.lens.height <= 0) return fail(VMHIP_ERR_ARGUMENT, "stage: empty image dimensions");
        if (in.n_ranges < 0 || (in.n_ranges > 0 && !in.ranges)) return fail(VMHIP_ERR_ARGUMENT, "stage: bad range table");
        if (classify && !E->layers.empty() && in.mesh->nn != E->nn)
            return fail(VMHIP_ERR_ARGUMENT, "stage: the mesh's neighbour count does not match the network");
        int fmt = VMHIP_FMT_NONE, bpp = 0;
        if (classify) {
            if (!decode_fourcc(in.fourcc, &fmt, &bpp)) return fail(VMHIP_ERR_FORMAT, "Unsupported image format " + fourcc_text(in.fourcc));
            if (!in.image) return fail(VMHIP_ERR_ARGUMENT, "stage: classification needs an image");
        }
        hf.mesh = in.mesh;
        hf.first.resize(in.n_ranges);
        hf.prefix.resize(size_t(in.n_ranges) + 1);
        int64_t total = 0;
        int32_t last_end = 0;
        for (int r = 0; r < in.n_ranges; ++r) {
            const int32_t a = in.ranges[2 * r], e = in.ranges[2 * r + 1];
            if (a < last_end || e < a || e > in.mesh->n_nodes) return fail(VMHIP_ERR_ARGUMENT, "stage: ranges must be ascending, disjoint and inside the mesh");
            hf.first[r] = a;
            hf.prefix[r] = int32_t(total);
            total += e - a;
            last_end = e;
        }
        hf.prefix[in.n_ranges] = int32_t(total);
        if (total > 0x7fff0000) return fail(VMHIP_ERR_ARGUMENT, "stage: too many candidates");

        VmFrame& d = hf.dev;
        std::memset(&d, 0, sizeof(d));
        d.rays = in.mesh->d_rays;
        d.nbr = in.mesh->d_nbr;
        d.n_nodes = in.mesh->n_nodes;
        d.nn = in.mesh->nn;
        std::memcpy(d.Rco, in.Rco, sizeof(d.Rco));
        d.focal = in.lens.focal_length;
        d.centre_x = hf.centre[0] = in.lens.centre[0];
        d.centre_y = hf.centre[1] = in.lens.centre[1];
        vm_host_inverse_coefficients(in.lens.k, d.ik);
        d.width = in.lens.width;
        d.height = in.lens.height;
        d.projection = in.lens.projection;
        d.fmt = fmt;
        d.n_ranges = in.n_ranges;
        d.n_cand = int32_t(total);
        d.cand_tile0 = int32_t(cand_tiles);
        d.cand_tiles = int32_t((total + VMHIP_TILE - 1) / VMHIP_TILE);
        d.cand_base = d.cand_tile0 * VMHIP_TILE;
        d.row_tile0 = int32_t(row_tiles);
        d.row_tiles = total > 0 ? int32_t((total + 1 + VMHIP_TILE - 1) / VMHIP_TILE) : 0;
        d.row_base = d.row_tile0 * VMHIP_TILE;
        cand_tiles += d.cand_tiles;
        row_tiles += d.row_tiles;
        if (cand_tiles > 0x7fffff || row_tiles > 0x7fffff) return fail(VMHIP_ERR_ARGUMENT, "stage: batch too large");
        range_ints += size_t(in.n_ranges) * 2 + 1;
        if (classify) image_bytes += align_up(size_t(in.lens.width) * in.lens.height * bpp, 256);
        lookup_entries += size_t(in.mesh->n_nodes) + 1;
        max_cand = std::max(max_cand, size_t(total));
        widest_mesh = std::max(widest_mesh, uint64_t(in.mesh->n_nodes) * uint64_t(in.mesh->nn));
        nb_stride = std::max(nb_stride, in.mesh->nn);
        uniform_nn = (f == 0 || uniform_nn == in.mesh->nn) ? in.mesh->nn : 0;
    }
    /* Launch grids and table offsets are sized for at least the tiles in use. An engine that replays captured passes
     * keeps them when a later batch fits (a batch that does not gets an eighth of slack, so that a stream of frames
     * settles after a few batches); kernel-by-kernel launches take exactly the tiles in use. */
    auto grown = [&](size_t have, size_t need) {
        if (!E->use_graph) return need;
        if (need <= have) return need * 2 < have ? need : have; /* far smaller batches do not launch the old one's grids */
        return have == 0 ? need : (need + need / 8 + 7) / 8 * 8;
    };
    b->cap_cand_tiles = std::min<size_t>(grown(b->cap_cand_tiles, cand_tiles), 0x7fffff);
    b->cap_row_tiles = std::min<size_t>(grown(b->cap_row_tiles, row_tiles), 0x7fffff);
    b->live.n_cand_tiles = int32_t(cand_tiles), b->live.n_row_tiles = int32_t(row_tiles);
    cand_tiles = b->cap_cand_tiles, row_tiles = b->cap_row_tiles; /* from here on: what is allocated and launched */
    b->cand_total = cand_tiles * VMHIP_TILE;
    b->row_total = row_tiles * VMHIP_TILE;
    const size_t words = b->cand_total / 64;
    if (classify && E->use_bf16 && max_cand + 1 >= (size_t(1) << 24))
        return fail(VMHIP_ERR_CAPACITY, "stage: a frame of 2^24 rows or more is too large for the bf16 layers (32-bit byte offsets into a frame's rows)");

    /* device workspace */
    /* the tiles in use, then the frame descriptions */
    constexpr size_t LIVE_BYTES = 64;
    static_assert(sizeof(VmBatchLive) <= LIVE_BYTES, "the frame descriptions follow the live counts");
    HIP_TRY(b->d_frames.reserve(LIVE_BYTES + sizeof(VmFrame) * n_frames));
    /* the tile tables ({frame, first range} per candidate tile, frame per row tile: at offsets that depend on the grid
     * sizes only), then the range tables */
    const size_t ranges_at = align_up(2 * cand_tiles + row_tiles, 2), n_table_ints = ranges_at + std::max<size_t>(range_ints, 1);
    /* the number of ranges varies from frame to frame with nothing to bound it: room for twice as many, so that the
     * tables rarely move (their address is part of a captured pass) */
    HIP_TRY(b->d_ranges.reserve(sizeof(int32_t) * (n_table_ints + (E->use_graph ? range_ints + 1024 : 0))));
    HIP_TRY(b->d_images.reserve(std::max<size_t>(image_bytes, 256)));
    HIP_TRY(b->d_cand_px.reserve(sizeof(float2) * std::max<size_t>(b->cand_total, 1)));
    HIP_TRY(b->d_cand_g.reserve(4 * std::max<size_t>(b->cand_total, 1)));
    HIP_TRY(b->d_cand_keep.reserve(8 * std::max<size_t>(words, 1)));
    HIP_TRY(b->d_tile_count.reserve(4 * std::max<size_t>(cand_tiles, 1)));
    HIP_TRY(b->d_force_valid.reserve(8 * std::max<size_t>(words, 1)));
    HIP_TRY(b->d_force_keep.reserve(8 * std::max<size_t>(words, 1)));
    HIP_TRY(b->d_frame_V.reserve(8 * size_t(n_frames))); /* visible counts, then ambiguity counts */
    /* a frame without candidates has no tile that would write its count; the ambiguity counters start from zero, and the
     * last kernel of every pass leaves them so */
    HIP_TRY(hipMemsetAsync(b->d_frame_V.p, 0, 8 * size_t(n_frames), E->stream));
    {
        const size_t need = 8 * size_t(n_frames) + sizeof(int2) * size_t(n_frames) * vmhip_batch::AMB_HEAD + 16;
        if (need > b->h_pin_cap) {
            if (b->h_pin) HIP_TRY(hipHostFree(b->h_pin));
            b->h_pin = nullptr, b->h_pin_cap = 0;
            HIP_TRY(hipHostMalloc(&b->h_pin, need, hipHostMallocDefault));
            b->h_pin_cap = need;
            HIP_TRY(hipHostGetDevicePointer(&b->h_pin_dev, b->h_pin, 0));
        }
    }
    HIP_TRY(b->d_amb_list.reserve(sizeof(int2) * size_t(n_frames) * VMHIP_AMB_CAP));
    HIP_TRY(b->d_row_px.reserve(sizeof(float2) * std::max<size_t>(b->row_total, 1)));
    HIP_TRY(b->d_row_gidx.reserve(4 * std::max<size_t>(b->row_total, 1)));
    HIP_TRY(b->d_row_nb.reserve(4 * std::max<size_t>(b->row_total, 1) * nb_stride));
    const bool local_tables = classify && E->use_lds && nb_stride <= VMHIP_NBL_STRIDE;
    if (classify) {
        for (int i = 0; i < 2; ++i) HIP_TRY(b->d_act[i].reserve(4 * std::max<size_t>(b->row_total, 1) * E->max_width));
    }
    if (local_tables) {
        const size_t row_tiles = std::max<size_t>(b->row_total / VMHIP_TILE, 1);
        HIP_TRY(b->d_row_nbl.reserve(2 * std::max<size_t>(b->row_total, 1) * VMHIP_NBL_STRIDE));
        HIP_TRY(b->d_tile_halo.reserve(4 * row_tiles * VMHIP_HALO_MAX));
        HIP_TRY(b->d_tile_desc.reserve(sizeof(int4) * row_tiles));
    }
    const bool half_tables = classify && E->use_bf16 && nb_stride <= VMHIP_NBL_STRIDE;
    if (half_tables) {
        const size_t row_tiles = std::max<size_t>(b->row_total / VMHIP_TILE, 1);
        HIP_TRY(b->d_row_nbl_h.reserve(2 * std::max<size_t>(b->row_total, 1) * VMHIP_NBL_STRIDE));
        HIP_TRY(b->d_tile_note_h.reserve(4 * 2 * row_tiles * VMHIP_NOTE_WORDS));
        HIP_TRY(b->d_active_h.reserve(4 * (size_t(n_frames) + 1)));
    }
    HIP_TRY(b->d_lookup.reserve(sizeof(uint32_t) * lookup_entries));
    b->lookup_total = lookup_entries;
    if (!b->d_epoch.p) {
        HIP_TRY(b->d_epoch.reserve(256));
        HIP_TRY(hipMemsetAsync(b->d_epoch.p, 0, 256, E->stream));
        HIP_TRY(hipMemsetD32Async(reinterpret_cast<hipDeviceptr_t>(b->d_epoch.p), 1, 1, E->stream));
        b->epoch = 0;
    }
    /* a reverse-lookup entry: the run's stamp above the node's row. 24 bits of row serve every frame below 2^24
     * candidates and leave 255 runs between two clears of the table; a larger frame takes the bits it needs from the stamp */
    int row_bits = std::min(std::max(24, g_debug_stamp_row_bits.load()), 31);
    while (row_bits < 31 && (max_cand >> row_bits) != 0) ++row_bits;
    if (b->d_lookup.grew || row_bits != b->stamp_row_bits) {
        /* a fresh table, or one whose entries were split differently, holds no valid stamp: zero everywhere, and the
         * runs count from one again */
        HIP_TRY(hipMemsetAsync(b->d_lookup.p, 0, b->d_lookup.cap, E->stream));
        HIP_TRY(hipMemsetD32Async(reinterpret_cast<hipDeviceptr_t>(b->d_epoch.p), 1, 1, E->stream));
        b->epoch = 0;
        b->stamp_row_bits = row_bits;
    }

    /* fill in device pointers and upload */
    {
        const size_t need = LIVE_BYTES + align_up(sizeof(VmFrame) * size_t(n_frames), 64) + 4 * n_table_ints;
        if (need > b->h_stage_cap) {
            if (b->h_stage) HIP_TRY(hipHostFree(b->h_stage));
            b->h_stage = nullptr, b->h_stage_cap = 0;
            HIP_TRY(hipHostMalloc(&b->h_stage, need + need / 4, hipHostMallocDefault));
            b->h_stage_cap = need + need / 4;
        }
    }
    *static_cast<VmBatchLive*>(b->h_stage) = b->live;
    VmFrame* h_frames = reinterpret_cast<VmFrame*>(static_cast<char*>(b->h_stage) + LIVE_BYTES);
    int32_t* h_ranges = reinterpret_cast<int32_t*>(static_cast<char*>(b->h_stage) + LIVE_BYTES + align_up(sizeof(VmFrame) * size_t(n_frames), 64));
    size_t range_off = ranges_at, image_off = 0, lookup_off = 0;
    const uint8_t* run_src = nullptr; /* the run of adjoining images not yet copied */
    size_t run_dst = 0, run_bytes = 0;
    for (int f = 0; f < n_frames; ++f) {
        HostFrame& hf = b->frames[f];
        VmFrame& d = hf.dev;
        const int R = d.n_ranges;
        d.range_first = b->d_ranges.as<int32_t>() + range_off;
        std::copy(hf.first.begin(), hf.first.end(), h_ranges + range_off);
        range_off += R;
        d.range_prefix = b->d_ranges.as<int32_t>() + range_off;
        std::copy(hf.prefix.begin(), hf.prefix.end(), h_ranges + range_off);
        range_off += size_t(R) + 1;
        if (classify) {
            int fmt, bpp;
            decode_fourcc(frames[f].fourcc, &fmt, &bpp);
            const size_t bytes = size_t(d.width) * d.height * bpp;
            d.image = b->d_images.as<uint8_t>() + image_off;
            /* images that follow one another in the caller's memory (a ring of camera buffers in one allocation) and on
             * the device go up as one copy: a few large copies cross the bus faster than many small ones */
            const uint8_t* src = static_cast<const uint8_t*>(frames[f].image);
            if (run_bytes > 0 && src == run_src + run_bytes && image_off == run_dst + run_bytes) {
                run_bytes += bytes;
            }
            else {
                if (run_bytes > 0) HIP_TRY(hipMemcpyAsync(b->d_images.as<uint8_t>() + run_dst, run_src, run_bytes, hipMemcpyHostToDevice, E->stream));
                run_src = src, run_dst = image_off, run_bytes = bytes;
            }
            image_off += align_up(bytes, 256);
        }
        d.r_lookup = b->d_lookup.as<uint32_t>() + lookup_off;
        lookup_off += size_t(d.n_nodes) + 1;
        d.force_valid = b->d_force_valid.as<uint64_t>();
        d.force_keep = b->d_force_keep.as<uint64_t>();
        h_frames[f] = d;
        /* the tiles of this frame: a candidate tile's first candidate lies in range r, prefix[r] <= first < prefix[r + 1] */
        int32_t* const cand_info = h_ranges + 2 * size_t(d.cand_tile0);
        int r = 0;
        for (int t = 0; t < d.cand_tiles; ++t) {
            while (r + 1 < R && hf.prefix[size_t(r) + 1] <= int64_t(t) * VMHIP_TILE) ++r;
            cand_info[2 * t] = f;
            cand_info[2 * t + 1] = r;
        }
        std::fill_n(h_ranges + 2 * cand_tiles + size_t(d.row_tile0), size_t(d.row_tiles), f);
    }
    if (run_bytes > 0) HIP_TRY(hipMemcpyAsync(b->d_images.as<uint8_t>() + run_dst, run_src, run_bytes, hipMemcpyHostToDevice, E->stream));
    HIP_TRY(hipMemcpyAsync(b->d_frames.p, b->h_stage, LIVE_BYTES + sizeof(VmFrame) * n_frames, hipMemcpyHostToDevice, E->stream));
    HIP_TRY(hipMemcpyAsync(b->d_ranges.p, h_ranges, sizeof(int32_t) * n_table_ints, hipMemcpyHostToDevice, E->stream));
    HIP_TRY(hipMemsetAsync(b->d_force_valid.p, 0, 8 * std::max<size_t>(words, 1), E->stream));
    HIP_TRY(hipMemsetAsync(b->d_force_keep.p, 0, 8 * std::max<size_t>(words, 1), E->stream));
    b->h_force_valid.assign(std::max<size_t>(words, 1), 0);
    b->h_force_keep.assign(std::max<size_t>(words, 1), 0);
    /* a stage that waits returns with the caller's images read; one that does not leaves its copies on the stream,
     * ahead of the run's kernels: the tables they read live in h_stage, the images must stay as they are until the
     * run has been waited for */
    if (wait) HIP_TRY(hipStreamSynchronize(E->stream));
    b->stage_pending = !wait;

    VmBatchDev& D = b->dev;
    std::memset(&D, 0, sizeof(D)); /* padding too: a captured pass is matched against this struct byte by byte */
    D.live = b->d_frames.as<VmBatchLive>();
    D.frames = reinterpret_cast<const VmFrame*>(b->d_frames.as<char>() + LIVE_BYTES);
    D.n_frames = n_frames;
    D.n_cand_tiles = int32_t(cand_tiles);
    D.n_row_tiles = int32_t(row_tiles);
    D.cand_px = b->d_cand_px.as<float2>();
    D.cand_g = b->d_cand_g.as<int32_t>();
    D.cand_keep = b->d_cand_keep.as<uint64_t>();
    D.tile_count = b->d_tile_count.as<int32_t>();
    D.frame_V = b->d_frame_V.as<int32_t>();
    D.amb_count = b->d_frame_V.as<int32_t>() + n_frames;
    D.amb_list = b->d_amb_list.as<int2>();
    D.row_px = b->d_row_px.as<float2>();
    D.row_gidx = b->d_row_gidx.as<int32_t>();
    D.row_nb = b->d_row_nb.as<int32_t>();
    D.nb_stride = nb_stride;
    D.row_nbl = local_tables ? b->d_row_nbl.as<uint16_t>() : nullptr;
    D.tile_halo = local_tables ? b->d_tile_halo.as<uint32_t>() : nullptr;
    D.tile_desc = local_tables ? b->d_tile_desc.as<int4>() : nullptr;
    D.halo_cap = E->halo_cap;
    D.active_h = half_tables ? b->d_active_h.as<int32_t>() : nullptr;
    D.row_nbl_h = half_tables ? b->d_row_nbl_h.as<uint16_t>() : nullptr;
    D.tile_note_h = half_tables ? b->d_tile_note_h.as<uint32_t>() : nullptr;
    D.epoch = b->d_epoch.as<uint32_t>();
    D.stamp_row_bits = b->stamp_row_bits;
    D.uniform_nn = uniform_nn;
    D.cand_tile_info = reinterpret_cast<const int2*>(b->d_ranges.as<int32_t>());
    D.row_tile_frame = b->d_ranges.as<int32_t>() + 2 * cand_tiles;
    /* 32-bit byte offsets into a frame's part of every table the neighbourhood kernel touches (4-byte entries of the
     * mesh's neighbour table and of the output table, 16-byte rows of the tile-local table), unless one is too large */
    D.wide_offsets = (widest_mesh >= (1ull << 30) || (uint64_t(max_cand) + 1) * uint64_t(std::max(nb_stride, 4)) >= (1ull << 30) || g_debug_wide_offsets.load()) ? 1 : 0;
    D.flow_timeouts = b->d_epoch.as<unsigned int>() + 16; /* same zeroed block, a cache line of its own */
    D.amb_eps = g_debug_edge_band.load();
    D.px_error = g_debug_px_error.load();
    b->reruns = 0, b->overruled = 0, b->amb_seen = 0, b->amb_most = 0;
    b->h_V.assign(n_frames, 0);
    b->h_amb_count.assign(n_frames, 0);
    return VMHIP_OK;
}

struct Profiler {
    vmhip_batch* b;
    hipStream_t s;
    int slot = 0;
    bool wanted() const { return b->profile == 1 || (b->profile == 2 && slot < int(b->slot_wanted.size()) && b->slot_wanted[slot]); }
    hipError_t begin() {
        if (!wanted()) return hipSuccess;
        while (int(b->events.size()) < 2 * (slot + 1)) {
            hipEvent_t e;
            hipError_t r = hipEventCreate(&e);
            if (r != hipSuccess) return r;
            b->events.push_back(e);
        }
        return hipEventRecord(b->events[2 * slot], s);
    }
    hipError_t end(const char* name, int64_t units) {
        if (!b->profile) return hipSuccess;
        hipError_t r = wanted() ? hipEventRecord(b->events[2 * slot + 1], s) : hipSuccess;
        if (int(b->slot_names.size()) <= slot) {
            b->slot_names.resize(slot + 1);
            b->slot_units.resize(slot + 1);
        }
        b->slot_names[slot] = name;
        b->slot_units[slot] = units;
        ++slot;
        return r;
    }
};

int batch_enqueue(vmhip_batch* b) {
    vmhip_engine* E = b->engine;
    hipStream_t s = E->stream;
    VmBatchDev& D = b->dev;
    Profiler P{b, s};
    int64_t cands = 0, rows = 0;
    for (const HostFrame& hf : b->frames) cands += hf.dev.n_cand;
    rows = cands + int64_t(b->frames.size());

    HIP_TRY(P.begin());
    vm_launch_project(D, s);
    HIP_TRY(P.end("project", cands));
    HIP_TRY(P.begin());
    vm_launch_compact(D, b->d_act[0].as<float>(), b->classify, s);
    HIP_TRY(P.end(b->classify ? "compact_sample" : "compact", cands));
    /* the neighbourhood table - and, where the first layer is a thin one over the sampled rows, that layer with it */
    int first_layer = 0, cur = 0;
    bool fused = false;
    if (b->classify && !E->layers.empty() && E->layers[0].fuse_first && D.row_nbl) {
        const HostLayer& L = E->layers[0];
        VmLayerDev ld{L.c_in, L.c_out, L.slots, L.activation, L.d_w, L.d_b, L.d_w_mfma, L.in_bf16, L.out_bf16, L.arith_bf16, L.d_w_flow};
        const char* name = "neighbourhood";
        HIP_TRY(P.begin());
        fused = vm_launch_neighbourhood_conv(D, ld, b->d_act[0].as<float>(), b->d_act[1].as<float>(), s, &name) == 0;
        if (fused) {
            HIP_TRY(P.end(name, rows));
            first_layer = 1, cur = 1;
        }
    }
    if (!fused) {
        HIP_TRY(P.begin()); /* (a second begin of the same slot records its start event again) */
        vm_launch_neighbourhood(D, s);
        HIP_TRY(P.end("neighbourhood", rows));
    }
    if (b->classify && D.row_nbl_h) {
        HIP_TRY(P.begin());
        vm_launch_half_tables(D, s);
        HIP_TRY(P.end("half_tables", rows));
    }

    if (b->classify) {
        for (size_t li = size_t(first_layer); li < E->layers.size(); ++li) {
            const HostLayer& L = E->layers[li];
            VmLayerDev ld{L.c_in, L.c_out, L.slots, L.activation, L.d_w, L.d_b, L.d_w_mfma, L.in_bf16, L.out_bf16, L.arith_bf16, L.d_w_flow};
            const char* name = "conv";
            HIP_TRY(P.begin());
            int rc = -1;
            if (L.arith_bf16) rc = vm_launch_conv_bf16(D, ld, b->d_act[cur].p, b->d_act[cur ^ 1].p, s, &name);
            if (rc != 0 && !L.arith_bf16 && L.use_narrow && D.row_nbl) rc = vm_launch_conv_narrow(D, ld, b->d_act[cur].as<float>(), b->d_act[cur ^ 1].as<float>(), s, &name);
            if (rc != 0 && L.use_flow && D.row_nbl) rc = vm_launch_conv_flow(D, ld, b->d_act[cur].as<float>(), b->d_act[cur ^ 1].as<float>(), s, &name);
            if (rc != 0 && L.use_lds && D.row_nbl) rc = vm_launch_conv_lds(D, ld, b->d_act[cur].as<float>(), b->d_act[cur ^ 1].as<float>(), s, &name);
            if (rc != 0 && L.d_w_mfma && L.use_mfma) rc = vm_launch_conv_mfma(D, ld, b->d_act[cur].as<float>(), b->d_act[cur ^ 1].as<float>(), s, &name);
            /* the one-row-per-lane kernels only know fp32 rows */
            if (rc != 0 && !L.in_bf16 && !L.out_bf16 && !L.arith_bf16) rc = vm_launch_conv(D, ld, b->d_act[cur].as<float>(), b->d_act[cur ^ 1].as<float>(), s, &name);
            if (rc != 0) return fail(VMHIP_ERR_HIP, "no kernel could be launched for a layer");
            HIP_TRY(P.end(name, rows));
            cur ^= 1;
        }
        b->final_act = b->d_act[cur].as<float>();
    }
    b->n_slots = P.slot;
    HIP_TRY(hipGetLastError());
    return VMHIP_OK;
}

/* Re-decide, with the host's arithmetic, every candidate the device flagged as lying within the
 * ambiguity band of a screen edge. Returns the number of decisions that differ (those are written
 * into the force masks), or a negative status. */
/* the run's one download (visible counts, ambiguity counts, heads of the ambiguity lists, the convolution kernel's
 * count of waits that ran out) into the pinned landing area, behind the run's kernels */
int batch_request_verdict(vmhip_batch* b) {
    vmhip_engine* E = b->engine;
    const int n = int(b->frames.size());
    constexpr int HEAD = vmhip_batch::AMB_HEAD;
    /* a kernel stores them into the page-locked landing area: small copies would wait in the copy engine's queue behind
     * whatever another engine is downloading */
    int32_t* pin_counts = reinterpret_cast<int32_t*>(b->h_pin_dev);
    int2* pin_amb = reinterpret_cast<int2*>(pin_counts + 2 * n);
    uint32_t* pin_timeouts = reinterpret_cast<uint32_t*>(pin_amb + size_t(n) * HEAD);
    /* the barrier-free convolution kernel bounds its waits; a wait that ran out (never in a correct run) means
     * the results of this run cannot be trusted */
    const unsigned int* d_timeouts = (E->use_flow && b->classify) ? b->dev.flow_timeouts : nullptr;
    vm_launch_publish(b->d_frame_V.as<int32_t>(), 2 * n, b->d_amb_list.as<int2>(), VMHIP_AMB_CAP, HEAD, n, d_timeouts, b->dev.epoch, pin_counts, pin_amb, pin_timeouts, E->stream);
    HIP_TRY(hipGetLastError());
    return VMHIP_OK;
}

int batch_verify(vmhip_batch* b) {
    vmhip_engine* E = b->engine;
    const int n = int(b->frames.size());
    constexpr int HEAD = vmhip_batch::AMB_HEAD;
    int32_t* pin_counts = reinterpret_cast<int32_t*>(b->h_pin);
    int2* pin_amb = reinterpret_cast<int2*>(pin_counts + 2 * n);
    uint32_t* pin_timeouts = reinterpret_cast<uint32_t*>(pin_amb + size_t(n) * HEAD);
    unsigned int* d_timeouts = (E->use_flow && b->classify) ? b->dev.flow_timeouts : nullptr;
    HIP_TRY(hipStreamSynchronize(E->stream));
    if (*pin_timeouts != 0) {
        (void) hipMemset(d_timeouts, 0, 4);
        return fail(VMHIP_ERR_HIP, "run: a convolution wave gave up waiting for its tile; the results of this run were discarded");
    }
    std::copy(pin_counts, pin_counts + n, b->h_V.begin());
    std::copy(pin_counts + n, pin_counts + 2 * n, b->h_amb_count.begin());
    int changed = 0;
    for (int f = 0; f < n; ++f) {
        HostFrame& hf = b->frames[f];
        const VmFrame& d = hf.dev;
        if (d.n_cand == 0) {
            b->h_V[f] = 0;
            continue;
        }
        const int count = b->h_amb_count[f];
        if (count == 0) continue;
        b->amb_seen += count;
        b->amb_most = std::max<int64_t>(b->amb_most, count);
        const float* rays = hf.mesh->h_rays.data();
        auto redecide = [&](int p, int gpu_keep, bool force_all) {
            /* candidate slot -> global index */
            const int r = int(std::upper_bound(hf.prefix.begin(), hf.prefix.end() - 1, p) - hf.prefix.begin()) - 1;
            const int g = hf.first[r] + (p - hf.prefix[r]);
            const int keep = vm_host_on_screen(d.Rco, rays + size_t(g) * 3, d.projection, d.focal, hf.centre, d.ik, d.width, d.height, nullptr);
            if (keep != gpu_keep || force_all) {
                const size_t word = (size_t(d.cand_base) + p) >> 6;
                const uint64_t bit = 1ull << (p & 63);
                b->h_force_valid[word] |= bit;
                if (keep) b->h_force_keep[word] |= bit;
                else b->h_force_keep[word] &= ~bit;
                if (keep != gpu_keep) ++changed;
            }
        };
        if (count > VMHIP_AMB_CAP) {
            /* the list overflowed: decide the whole frame on the host (slow, never seen with real lenses) */
            for (int p = 0; p < d.n_cand; ++p) redecide(p, -1, true);
        }
        else {
            const int2* list = pin_amb + size_t(f) * HEAD;
            if (count > HEAD) { /* more than the head that came with the counts */
                b->h_amb.resize(count);
                HIP_TRY(hipMemcpy(b->h_amb.data(), b->d_amb_list.as<int2>() + size_t(f) * VMHIP_AMB_CAP, sizeof(int2) * count, hipMemcpyDeviceToHost));
                list = b->h_amb.data();
            }
            for (int i = 0; i < count; ++i) redecide(list[i].x, list[i].y, false);
        }
    }
    if (changed > 0) {
        b->overruled += changed;
        ++b->reruns;
        const size_t words = std::max<size_t>(b->cand_total / 64, 1);
        HIP_TRY(hipMemcpyAsync(b->d_force_valid.p, b->h_force_valid.data(), 8 * words, hipMemcpyHostToDevice, E->stream));
        HIP_TRY(hipMemcpyAsync(b->d_force_keep.p, b->h_force_keep.data(), 8 * words, hipMemcpyHostToDevice, E->stream));
        HIP_TRY(hipStreamSynchronize(E->stream));
    }
    return changed;
}

/* puts one pass over the staged frames, and the download of its verdict, on the engine's stream */
int batch_launch(vmhip_batch* b) {
    vmhip_engine* E = b->engine;
    if (b->epoch >= (0xffffffffu >> b->stamp_row_bits)) { /* the stamp has used all its bits: old stamps could look current again */
        HIP_TRY(hipMemsetAsync(b->d_lookup.p, 0, b->d_lookup.cap, E->stream));
        HIP_TRY(hipMemsetD32Async(reinterpret_cast<hipDeviceptr_t>(b->d_epoch.p), 1, 1, E->stream));
        b->epoch = 0;
    }
    /* The pass runs with stamp epoch + 1, which is what the device word holds: the last kernel of a pass advances the
     * word, so the host's mirror advances once that kernel has been queued. */
    int rc = VMHIP_OK;
    /* profile mode 2 (events around the launches of one kernel only) is captured too: its event records become nodes of the graph */
    if (E->use_graph && b->profile != 1) {
        vmhip_batch::GraphKey key;
        std::memset(&key, 0, sizeof(key));
        std::memcpy(&key.dev, &b->dev, sizeof(VmBatchDev));
        key.act[0] = b->d_act[0].p, key.act[1] = b->d_act[1].p;
        key.pin = b->h_pin_dev;
        key.classify = b->classify, key.profile = b->profile;
        if (b->graph_exec && std::memcmp(&key, &b->graph_key, sizeof(key)) != 0) b->drop_graph(); /* an address, a grid or the mode has changed */
        if (b->graph_exec || b->eager_runs >= 1) {
            if (!b->graph_exec) {
                /* Capture the kernel sequence (kernels only: the clears are a kernel too, no memset nodes). A pass has been
                 * launched kernel by kernel before, so every kernel's one-time attribute set-up is done. */
                HIP_TRY(hipStreamBeginCapture(E->stream, hipStreamCaptureModeThreadLocal));
                rc = batch_enqueue(b);
                if (rc == VMHIP_OK) rc = batch_request_verdict(b); /* the pass's last kernel is part of the graph */
                hipError_t e = hipStreamEndCapture(E->stream, &b->graph);
                if (rc != VMHIP_OK || e != hipSuccess) {
                    if (e == hipSuccess && b->graph) (void) hipGraphDestroy(b->graph);
                    b->graph = nullptr;
                    if (rc != VMHIP_OK) return rc;
                    HIP_TRY(e);
                }
                if (hipGraphInstantiate(&b->graph_exec, b->graph, nullptr, nullptr, 0) != hipSuccess) {
                    b->graph_exec = nullptr;
                    b->drop_graph();
                    return fail(VMHIP_ERR_HIP, "run: the captured pass could not be instantiated");
                }
                std::memcpy(&b->graph_key, &key, sizeof(key));
                ++b->graph_captures;
            }
            HIP_TRY(hipGraphLaunch(b->graph_exec, E->stream));
            ++b->graph_launches;
            ++b->epoch;
            return VMHIP_OK;
        }
    }
    rc = batch_enqueue(b);
    if (rc != VMHIP_OK) return rc;
    rc = batch_request_verdict(b);
    if (rc != VMHIP_OK) return rc;
    ++b->eager_runs;
    ++b->eager_launches;
    ++b->epoch;
    return VMHIP_OK;
}

/* waits for a launched pass; repeats it (a few times at most) while the host overrules edge decisions of the device */
int batch_complete(vmhip_batch* b) {
    for (int attempt = 0; attempt < 4; ++attempt) {
        int rc = batch_verify(b);
        if (rc < 0) return rc;
        if (rc == 0) {
            b->have_run = true;
            b->stage_pending = false; /* the stream has been waited for */
            ++b->run_serial;
            return VMHIP_OK;
        }
        if (attempt == 3) break;
        rc = batch_launch(b);
        if (rc != VMHIP_OK) return rc;
    }
    return fail(VMHIP_ERR_HIP, "run: edge decisions did not settle");
}

int batch_run(vmhip_batch* b) {
    if (b->frames.empty()) return fail(VMHIP_ERR_ARGUMENT, "run: nothing staged");
    if (b->in_flight) return fail(VMHIP_ERR_ARGUMENT, "run: a run of this batch is still in flight (vmhip_batch_wait first)");
    if (b->fetching) return fail(VMHIP_ERR_ARGUMENT, "run: a fetch of this batch is still in flight (vmhip_batch_fetch_wait first)");
    b->have_run = false; /* a run that fails leaves nothing to fetch */
    const int rc = batch_launch(b);
    if (rc != VMHIP_OK) return rc;
    return batch_complete(b);
}

/* the copies of a fetch, on the engine's stream; the caller waits for the stream */
int batch_fetch_enqueue(vmhip_batch* b, vmhip_result* results) {
    if (!b->have_run) return fail(VMHIP_ERR_ARGUMENT, "fetch: no completed run");
    if (!results) return fail(VMHIP_ERR_ARGUMENT, "fetch: null results");
    if (b->fetching) return fail(VMHIP_ERR_ARGUMENT, "fetch: a fetch of this batch is still in flight (vmhip_batch_fetch_wait first)");
    vmhip_engine* E = b->engine;
    hipStream_t s = E->stream;
    const int n = int(b->frames.size());
    const int stride = b->dev.nb_stride;
    const int C = E->n_classes;
    for (int f = 0; f < n; ++f) {
        const VmFrame& d = b->frames[f].dev;
        vmhip_result& R = results[f];
        const int V = b->h_V[f];
        R.n_visible = V;
        if (V == 0) continue;
        if (R.capacity < V) return fail(VMHIP_ERR_CAPACITY, "fetch: result capacity is smaller than the visible node count");
        const size_t base = size_t(d.row_base);
        if (R.pixel_coordinates)
            HIP_TRY(hipMemcpyAsync(R.pixel_coordinates, b->dev.row_px + base, sizeof(float2) * V, hipMemcpyDeviceToHost, s));
        if (R.global_indices)
            HIP_TRY(hipMemcpyAsync(R.global_indices, b->dev.row_gidx + base, 4 * size_t(V), hipMemcpyDeviceToHost, s));
        if (R.neighbourhood) {
            if (stride == d.nn)
                HIP_TRY(hipMemcpyAsync(R.neighbourhood, b->dev.row_nb + base * stride, 4 * size_t(V + 1) * d.nn, hipMemcpyDeviceToHost, s));
            else
                HIP_TRY(hipMemcpy2DAsync(R.neighbourhood, 4 * size_t(d.nn), b->dev.row_nb + base * stride, 4 * size_t(stride),
                                         4 * size_t(d.nn), size_t(V + 1), hipMemcpyDeviceToHost, s));
        }
        if (R.classifications && b->classify)
            HIP_TRY(hipMemcpyAsync(R.classifications, b->final_act + base * C, 4 * size_t(V + 1) * C, hipMemcpyDeviceToHost, s));
    }
    return VMHIP_OK;
}

/* where frame f's arrays lie in the block of a packed fetch: pixels, indices, neighbourhood, classifications, each at a
 * multiple of 256 bytes; returns the block's size */
size_t packed_layout(const vmhip_batch* b, std::vector<size_t>* offsets) {
    const int n = int(b->frames.size());
    const int C = b->engine->n_classes;
    size_t at = 0;
    if (offsets) offsets->assign(size_t(n) * 4, 0);
    for (int f = 0; f < n; ++f) {
        const size_t V = size_t(b->h_V[f]);
        if (V == 0) continue;
        const size_t sizes[4] = {8 * V, 4 * V, 4 * (V + 1) * size_t(b->frames[f].dev.nn), b->classify ? 4 * (V + 1) * size_t(C) : 0};
        for (int k = 0; k < 4; ++k) {
            if (offsets) (*offsets)[size_t(f) * 4 + k] = at;
            at += align_up(sizes[k], 256);
        }
    }
    return at;
}

/* vmhip_batch_fetch_packed_async: one kernel gathers every frame's arrays into one device block, one copy brings it home */
int batch_fetch_packed_enqueue(vmhip_batch* b, void* block, size_t bytes, vmhip_result* results) {
    if (!b->have_run) return fail(VMHIP_ERR_ARGUMENT, "fetch: no completed run");
    if (!results || !block) return fail(VMHIP_ERR_ARGUMENT, "fetch_packed: null block or results");
    if (b->fetching) return fail(VMHIP_ERR_ARGUMENT, "fetch: a fetch of this batch is still in flight (vmhip_batch_fetch_wait first)");
    vmhip_engine* E = b->engine;
    hipStream_t s = E->stream;
    const int n = int(b->frames.size());
    const int C = E->n_classes;
    std::vector<size_t> offsets;
    const size_t total = packed_layout(b, &offsets);
    if (bytes < total) return fail(VMHIP_ERR_CAPACITY, "fetch_packed: the block is smaller than vmhip_batch_fetch_packed_size says");
    const size_t table_bytes = sizeof(VmPackSegment) * size_t(n) * 4;
    if (table_bytes > b->h_pack_cap) {
        if (b->h_pack) HIP_TRY(hipHostFree(b->h_pack));
        b->h_pack = nullptr, b->h_pack_cap = 0;
        HIP_TRY(hipHostMalloc(&b->h_pack, table_bytes, hipHostMallocDefault));
        b->h_pack_cap = table_bytes;
    }
    VmPackSegment* seg = static_cast<VmPackSegment*>(b->h_pack);
    int n_seg = 0, n_chunks = 0;
    uint8_t* host = static_cast<uint8_t*>(block);
    for (int f = 0; f < n; ++f) {
        const VmFrame& d = b->frames[f].dev;
        vmhip_result& R = results[f];
        const size_t V = size_t(b->h_V[f]);
        R.capacity = R.n_visible = int32_t(V);
        R.pixel_coordinates = nullptr, R.global_indices = nullptr, R.neighbourhood = nullptr, R.classifications = nullptr;
        if (V == 0) continue;
        const size_t base = size_t(d.row_base), stride = size_t(b->dev.nb_stride);
        const size_t* at = &offsets[size_t(f) * 4];
        auto add = [&](const void* src, size_t dst_offset, size_t nbytes, size_t row_bytes, size_t src_stride) {
            seg[n_seg++] = VmPackSegment{static_cast<const uint8_t*>(src), dst_offset, nbytes, row_bytes, src_stride, n_chunks};
            n_chunks += int((nbytes + VM_PACK_CHUNK - 1) / VM_PACK_CHUNK);
        };
        add(b->dev.row_px + base, at[0], 8 * V, 8, 8);
        add(b->dev.row_gidx + base, at[1], 4 * V, 4, 4);
        add(b->dev.row_nb + base * stride, at[2], 4 * (V + 1) * size_t(d.nn), 4 * size_t(d.nn), 4 * stride);
        R.pixel_coordinates = reinterpret_cast<float*>(host + at[0]);
        R.global_indices = reinterpret_cast<int32_t*>(host + at[1]);
        R.neighbourhood = reinterpret_cast<int32_t*>(host + at[2]);
        if (b->classify) {
            add(b->final_act + base * C, at[3], 4 * (V + 1) * size_t(C), 4 * size_t(C), 4 * size_t(C));
            R.classifications = reinterpret_cast<float*>(host + at[3]);
        }
    }
    if (total == 0) return VMHIP_OK;
    HIP_TRY(b->d_fetch_packed.reserve(total));
    /* the kernel reads the table where it lies, in page-locked host memory: an upload would wait in the copy engine's
     * queue behind the images another engine is staging. The table is not touched again before vmhip_batch_fetch_wait. */
    void* seg_dev = nullptr;
    HIP_TRY(hipHostGetDevicePointer(&seg_dev, seg, 0));
    vm_launch_fetch_pack(static_cast<const VmPackSegment*>(seg_dev), n_seg, n_chunks, b->d_fetch_packed.p, s);
    HIP_TRY(hipGetLastError());
    HIP_TRY(hipMemcpyAsync(block, b->d_fetch_packed.p, total, hipMemcpyDeviceToHost, s));
    return VMHIP_OK;
}

int batch_fetch(vmhip_batch* b, vmhip_result* results) {
    const int rc = batch_fetch_enqueue(b, results);
    /* wait also when a copy could not be queued: the ones before it write into the caller's arrays */
    const hipError_t e = hipStreamSynchronize(b->engine->stream);
    if (rc != VMHIP_OK) return rc;
    HIP_TRY(e);
    return VMHIP_OK;
}

int ensure_scratch(vmhip_engine* E) {
    if (!E->scratch) {
        E->scratch = new vmhip_batch();
        E->scratch->engine = E;
    }
    return VMHIP_OK;
}

}  // namespace

int vm_set_error(int code, const char* message) { return fail(code, message); }
bool vm_decode_fourcc(uint32_t fourcc, int* fmt, int* bytes_per_pixel) { return decode_fourcc(fourcc, fmt, bytes_per_pixel); }
void vm_debug_knobs(double* projection_error, double* edge_band) {
    *projection_error = double(g_debug_px_error.load());
    *edge_band = double(g_debug_edge_band.load());
}

extern "C" {

const char* vmhip_last_error(void) { return g_error.c_str(); }

int vmhip_engine_create(const vmhip_network* net, int32_t n_neighbours, int32_t precision, vmhip_engine** out) {
    if (!out) return fail(VMHIP_ERR_ARGUMENT, "engine_create: null output");
    *out = nullptr;
    if (n_neighbours < 0 || n_neighbours > 16) return fail(VMHIP_ERR_ARGUMENT, "engine_create: unsupported neighbour count");
    if (precision == VMHIP_FP64)
        return fail(VMHIP_ERR_ARGUMENT, "engine_create: a double engine takes double weights: use vmhip_engine_create_f64 and the other _f64 entry points");
    if (precision != VMHIP_FP32 && precision != VMHIP_BF16 && precision != VMHIP_SPLIT) return fail(VMHIP_ERR_ARGUMENT, "engine_create: unknown precision");
    int n_dev = 0;
    HIP_TRY(hipGetDeviceCount(&n_dev));
    if (n_dev <= 0) return fail(VMHIP_ERR_HIP, "engine_create: no HIP device");

    vmhip_engine* E = new vmhip_engine();
    E->nn = n_neighbours;
    E->precision = precision;
    auto bail = [&](int code, const std::string& msg) {
        vmhip_engine_destroy(E);
        return fail(code, msg);
    };
    int width = 4;
    int li = 0;
    for (int g = 0; net && g < net->n_groups; ++g) {
        if (net->group_sizes[g] <= 0) return bail(VMHIP_ERR_ARGUMENT, "engine_create: empty convolutional group");
        for (int l = 0; l < net->group_sizes[g]; ++l, ++li) {
            const vmhip_layer& L = net->layers[li];
            const int slots = l == 0 ? n_neighbours + 1 : 1;
            if (L.n_in != slots * width || L.n_out <= 0 || !L.weights || !L.biases)
                return bail(VMHIP_ERR_ARGUMENT, "engine_create: layer " + std::to_string(li) + " expects " + std::to_string(slots * width)
                                                  + " inputs, has " + std::to_string(L.n_in));
            if (L.activation < VMHIP_SELU || L.activation > VMHIP_TANH) return bail(VMHIP_ERR_ARGUMENT, "engine_create: unknown activation");
            HostLayer H;
            H.c_in = width, H.c_out = L.n_out, H.slots = slots, H.activation = L.activation;
            H.h_w.assign(L.weights, L.weights + size_t(L.n_in) * L.n_out);
            H.h_b.assign(L.biases, L.biases + size_t(L.n_out));
            if (hipMalloc(&H.d_w, 4 * size_t(L.n_in) * L.n_out) != hipSuccess || hipMalloc(&H.d_b, 4 * size_t(L.n_out)) != hipSuccess)
                return bail(VMHIP_ERR_HIP, "engine_create: out of device memory");
            E->layers.push_back(H);
            if (hipMemcpy(H.d_w, L.weights, 4 * size_t(L.n_in) * L.n_out, hipMemcpyHostToDevice) != hipSuccess
                || hipMemcpy(H.d_b, L.biases, 4 * size_t(L.n_out), hipMemcpyHostToDevice) != hipSuccess)
                return bail(VMHIP_ERR_HIP, "engine_create: weight upload failed");
            width = L.n_out;
            E->max_width = std::max(E->max_width, width);
        }
    }
    E->n_classes = width;

    /* Row formats and arithmetic per layer. fp32 engine: everything fp32. bf16 engine: the layers that conv_bf16.hip
     * has a kernel for (64 -> 64) run on the bf16 matrix instructions with fp32 accumulation and weights as hi + lo
     * pairs of bf16. The rows such a layer reads are stored either as bf16 (half the bytes, one bf16 rounding of
     * that layer's inputs against the fp32 result) or as hi + lo pairs of bf16 (the bytes of an fp32 row, no
     * bf16-sized error). One rounded boundary moves the final probabilities of a 6 x 64 network by up to ~4.6e-3,
     * n of them by about sqrt(n) times that (two: 7.2e-3, all five: 1.03e-2, measured on full-size frames), so to stay
     * inside the 1e-2 gate with margin every second boundary between bf16 layers is rounded and never more than two
     * in a network. What one rounding costs grows with the depth of the network, wherever it sits (a single rounded
     * boundary: 5-7e-3 with six 64-wide layers, 0.8-1.5e-2 with ten, 1.1-2.2e-2 with fourteen, on random networks), so
     * a network with more than five bf16 layers gets none: all its boundaries are hi + lo pairs (1e-4 with ten layers,
     * 1.6e-4 with fourteen). A bf16 layer behind a kernel that cannot write hi + lo rows reads fp32 rows and splits
     * them in registers. VMHIP_BF16_ROUNDED=n (at most n rounded boundaries) and VMHIP_BF16_ROUNDED_AT=mask (bit l:
     * the rows entering layer l) override the plan for measurements. */
    {
        /* VMHIP_CONV_KERNEL selects the kernel family for A/B runs: "rows" = one row per lane, "mfma" = matrix
         * cores gathering into registers, "lds" = matrix cores gathering from LDS (rows staged through registers),
         * "flow" = the same with rows loaded straight into LDS and no barriers in the tile loop,
         * wherever the shape has an instantiation; unset = the fastest measured kernel per layer shape */
        const char* pick = getenv("VMHIP_CONV_KERNEL");
        const bool rows_only = pick && std::string(pick) == "rows";
        const bool allow_lds = !rows_only && !(pick && std::string(pick) == "mfma");
        const bool force_lds = pick && std::string(pick) == "lds";
        const bool force_flow = pick && std::string(pick) == "flow";
        if (const char* g = getenv("VMHIP_GRAPH")) E->use_graph = atoi(g) != 0;
        if (const char* cap = getenv("VMHIP_HALO_CAP")) E->halo_cap = std::min(std::max(atoi(cap), 0), VMHIP_HALO_MAX);
        const int n = int(E->layers.size());
        std::vector<int> bf(n + 1, VM_ROWS_F32); /* bf[l] = format of the rows entering layer l; bf[n] = final output (fp32) */
        std::vector<int> ar(n, 0);               /* ar[l] = layer l uses the bf16 matrix instructions */
        if ((precision == VMHIP_BF16 || precision == VMHIP_SPLIT) && !rows_only) {
            for (int l = 0; l < n; ++l)
                ar[l] = (E->layers[l].slots - 1 <= VMHIP_NBL_STRIDE && vm_bf16_supported(E->layers[l].c_in, E->layers[l].c_out, E->layers[l].slots)) ? 1 : 0;
            int eligible = 0, rounded = 0;
            int n_bf16 = 0;
            for (int l = 0; l < n; ++l) n_bf16 += ar[l];
            int max_rounded = (n_bf16 <= 5 && precision == VMHIP_BF16) ? 2 : 0; /* VMHIP_SPLIT: every boundary as pairs */
            /* the split engine's contract has no rounded boundary: the measurement overrides are for the bf16 engine only */
            const bool overridable = precision == VMHIP_BF16;
            if (precision == VMHIP_SPLIT && n_bf16 > 10)
                return bail(VMHIP_ERR_ARGUMENT, "engine_create: VMHIP_SPLIT keeps its accuracy for up to ten 64-wide layers; use VMHIP_FP32 for this network");
            if (const char* r = getenv("VMHIP_BF16_ROUNDED")) max_rounded = overridable ? std::max(atoi(r), 0) : max_rounded;
            for (int l = 1; l < n; ++l) {
                if (!ar[l]) continue;
                ++eligible;
                const HostLayer& P = E->layers[l - 1];
                const bool splits = ar[l - 1] || (allow_lds && P.slots - 1 <= VMHIP_NBL_STRIDE && vm_lds_supported(P.c_in, P.c_out, P.slots, VM_ROWS_BF16X2));
                if (!splits) continue; /* the layer before writes fp32 rows */
                bool round_here = ar[l - 1] && eligible % 2 == 0 && rounded < max_rounded;
                if (const char* at = getenv("VMHIP_BF16_ROUNDED_AT"))
                    if (overridable) round_here = ar[l - 1] && ((strtoul(at, nullptr, 0) >> l) & 1ul);
                if (round_here) bf[l] = VM_ROWS_BF16, ++rounded;
                else bf[l] = VM_ROWS_BF16X2;
            }
        }
        auto arith = [&](int l) { return ar[l]; };
        for (int l = 0; l < n; ++l) {
            HostLayer& H = E->layers[l];
            H.in_bf16 = bf[l], H.out_bf16 = bf[l + 1], H.arith_bf16 = arith(l);
            const bool plain = !H.in_bf16 && !H.out_bf16 && !H.arith_bf16;
            H.use_mfma = !rows_only && plain && vm_mfma_supported(H.c_in, H.c_out, H.slots);
            H.use_lds = allow_lds && !H.in_bf16 && !H.arith_bf16 && H.slots - 1 <= VMHIP_NBL_STRIDE && vm_lds_supported(H.c_in, H.c_out, H.slots, H.out_bf16);
            E->use_bf16 = E->use_bf16 || H.arith_bf16;
            /* Measured on the 16-frame 1280x1024 workload: the LDS gather is the faster matrix-core kernel on every
             * shape it has (32->32: 157 us against 166 us, 32->16: 89 against 122, 4->16: 29 against 44); only the
             * 2- and 3-class output layers are quicker with one row per lane (46 us against 56 us). */
            if (H.use_lds && !force_lds && H.c_out < 4) H.use_lds = false;
            if (H.out_bf16 && !H.arith_bf16 && !H.use_lds) return bail(VMHIP_ERR_ARGUMENT, "engine_create: no kernel writes the rows the next layer was planned to read");
            /* the barrier-free variant of the LDS gather is the faster one where the matrix pipe is the limit
             * (32 -> 32: 147 us against 158 us, 32 -> 16: 93 against 99) and makes no difference for 16-wide input */
            H.use_flow = (force_flow || (allow_lds && !force_lds && H.c_in >= 32)) && plain && H.slots - 1 <= VMHIP_NBL_STRIDE
                         && vm_flow_supported(H.c_in, H.c_out, H.slots);
            /* class layers (at most four output channels): the 4x4x1 matrix instruction, unless a family is forced */
            H.use_narrow = allow_lds && !force_lds && plain && H.slots - 1 <= VMHIP_NBL_STRIDE
                           && vm_narrow_supported(H.c_in, H.c_out, H.slots);
            E->use_lds = E->use_lds || H.use_lds || H.use_flow || H.use_narrow;
            /* the first layer inside the neighbourhood kernel (VMHIP_FUSE_FIRST=0: as a launch of its own, for comparisons) */
            {
                const char* fuse = getenv("VMHIP_FUSE_FIRST");
                H.fuse_first = l == 0 && plain && H.use_lds && !pick && !(fuse && atoi(fuse) == 0) && n_neighbours <= VMHIP_NBL_STRIDE
                               && vm_neighbourhood_conv_supported(H.c_in, H.c_out, H.slots, H.activation);
            }
            E->use_flow = E->use_flow || H.use_flow;
            if (H.arith_bf16) {
                std::vector<unsigned char> wp(vm_bf16_weight_bytes(H.c_in, H.c_out, H.slots));
                vm_bf16_permute_weights(H.h_w.data(), H.c_in, H.c_out, H.slots, H.out_bf16, wp.data());
                if (hipMalloc(&H.d_w_mfma, wp.size()) != hipSuccess) return bail(VMHIP_ERR_HIP, "engine_create: out of device memory");
                if (hipMemcpy(H.d_w_mfma, wp.data(), wp.size(), hipMemcpyHostToDevice) != hipSuccess)
                    return bail(VMHIP_ERR_HIP, "engine_create: weight upload failed");
            }
            else if (H.use_mfma || H.use_lds || H.use_flow) {
                if (H.use_lds && H.out_bf16 == VM_ROWS_BF16X2) {
                    /* The one kernel that writes hi + lo rows without reading them keeps a lane's output values next to
                     * each other in the row: matrix column cb * 16 + q * 4 + v stands for channel q * 4 * CB + cb * 4 + v
                     * (conv_lds.hip), so weights and biases go to the device with their columns in that order. No other
                     * kernel can take this layer, so none sees the biases out of order. */
                    const int c_out = H.c_out, column_blocks = c_out / 16;
                    auto channel_of = [&](int column) { return ((column % 16) / 4) * (4 * column_blocks) + (column / 16) * 4 + column % 4; };
                    std::vector<float> w(H.h_w.size()), bias(H.h_b.size());
                    for (size_t k = 0; k < H.h_w.size() / size_t(c_out); ++k)
                        for (int column = 0; column < c_out; ++column) w[k * c_out + column] = H.h_w[k * c_out + channel_of(column)];
                    for (int column = 0; column < c_out; ++column) bias[column] = H.h_b[channel_of(column)];
                    H.h_w.swap(w);
                    if (hipMemcpy(H.d_b, bias.data(), 4 * bias.size(), hipMemcpyHostToDevice) != hipSuccess)
                        return bail(VMHIP_ERR_HIP, "engine_create: weight upload failed");
                }
                std::vector<unsigned char> wp(vm_mfma_weight_bytes(H.c_in, H.c_out, H.slots));
                vm_mfma_permute_weights(H.h_w.data(), H.c_in, H.c_out, H.slots, wp.data());
                if (hipMalloc(&H.d_w_mfma, wp.size()) != hipSuccess) return bail(VMHIP_ERR_HIP, "engine_create: out of device memory");
                if (hipMemcpy(H.d_w_mfma, wp.data(), wp.size(), hipMemcpyHostToDevice) != hipSuccess)
                    return bail(VMHIP_ERR_HIP, "engine_create: weight upload failed");
                if (H.use_flow) {
                    std::vector<float> wf(wp.size() / sizeof(float));
                    vm_flow_order_weights(reinterpret_cast<const float*>(wp.data()), H.c_in, H.c_out, H.slots, wf.data());
                    if (hipMalloc(&H.d_w_flow, wp.size()) != hipSuccess) return bail(VMHIP_ERR_HIP, "engine_create: out of device memory");
                    if (hipMemcpy(H.d_w_flow, wf.data(), wp.size(), hipMemcpyHostToDevice) != hipSuccess)
                        return bail(VMHIP_ERR_HIP, "engine_create: weight upload failed");
                }
            }
            H.h_w.clear();
            H.h_w.shrink_to_fit();
            H.h_b.clear();
        }
    }
    if (hipStreamCreateWithFlags(&E->stream, hipStreamNonBlocking) != hipSuccess) return bail(VMHIP_ERR_HIP, "engine_create: stream creation failed");
    /* Every engine owns a stream, and the runtime spreads the process's streams over GPU_MAX_HW_QUEUES hardware queues (4
     * unless the environment says otherwise). Streams that share a queue take turns: three engines in rotation lose 40 %
     * (2.55 ms per batch instead of 1.82) when a fourth engine's stream makes two of them share. Said once. */
    {
        const char* q = getenv("GPU_MAX_HW_QUEUES");
        const int queues = q && atoi(q) > 0 ? atoi(q) : 4;
        static std::atomic<bool> said{false};
        if (++g_live_engines + 1 > queues && !said.exchange(true)) /* + 1: the default stream */
            fprintf(stderr, "libvisualmesh_hip: %d engines are alive, each with a stream of its own, on %d hardware queues: engines that work at the same "
                            "time will take turns; set GPU_MAX_HW_QUEUES to at least the number of engines + 1 before the process starts\n",
                    g_live_engines.load(), queues);
    }
    E->counted = true;
    *out = E;
    return VMHIP_OK;
}

void vmhip_engine_destroy(vmhip_engine* E) {
    if (!E) return;
    if (E->scratch) vmhip_batch_destroy(E->scratch);
    for (HostLayer& L : E->layers) {
        if (L.d_w) (void) hipFree(L.d_w);
        if (L.d_b) (void) hipFree(L.d_b);
        if (L.d_w_mfma) (void) hipFree(L.d_w_mfma);
        if (L.d_w_flow) (void) hipFree(L.d_w_flow);
    }
    if (E->stream) (void) hipStreamDestroy(E->stream);
    if (E->counted) --g_live_engines;
    delete E;
}

int32_t vmhip_engine_n_classes(const vmhip_engine* E) { return E ? E->n_classes : 0; }

int vmhip_mesh_upload(const float* rays, const int32_t* neighbours, int32_t n_nodes, int32_t n_neighbours, vmhip_mesh** out) {
    if (!out) return fail(VMHIP_ERR_ARGUMENT, "mesh_upload: null output");
    *out = nullptr;
    if (!rays || !neighbours || n_nodes <= 0 || n_neighbours <= 0 || n_neighbours > 16)
        return fail(VMHIP_ERR_ARGUMENT, "mesh_upload: bad arguments");
    for (size_t i = 0; i < size_t(n_nodes) * n_neighbours; ++i)
        if (neighbours[i] < 0 || neighbours[i] > n_nodes) return fail(VMHIP_ERR_ARGUMENT, "mesh_upload: neighbour index outside [0, n_nodes]");
    vmhip_mesh* M = new vmhip_mesh();
    M->n_nodes = n_nodes;
    M->nn = n_neighbours;
    /* the one place every caller of vmhip_project_noalloc has passed through on its device: resolve that entry
     * point's workspace here, so that the entry point itself has nothing left to set up */
    if (hipGetDevice(&M->device) != hipSuccess || vm_noalloc_setup() != hipSuccess) {
        delete M;
        return fail(VMHIP_ERR_HIP, "mesh_upload: no usable device");
    }
    M->h_rays.assign(rays, rays + size_t(n_nodes) * 3);
    const size_t rb = sizeof(float) * 3 * size_t(n_nodes), nb = sizeof(int32_t) * size_t(n_nodes) * n_neighbours;
    if (hipMalloc(&M->d_rays, rb) != hipSuccess || hipMalloc(&M->d_nbr, nb) != hipSuccess
        || hipMemcpy(M->d_rays, rays, rb, hipMemcpyHostToDevice) != hipSuccess
        || hipMemcpy(M->d_nbr, neighbours, nb, hipMemcpyHostToDevice) != hipSuccess) {
        vmhip_mesh_release(M);
        return fail(VMHIP_ERR_HIP, "mesh_upload: device allocation or copy failed");
    }
    *out = M;
    return VMHIP_OK;
}

void vmhip_mesh_release(vmhip_mesh* M) {
    if (!M) return;
    if (M->d_rays) (void) hipFree(M->d_rays);
    if (M->d_nbr) (void) hipFree(M->d_nbr);
    if (M->d_tree) (void) hipFree(M->d_tree);
    delete M;
}

int vmhip_mesh_attach_tree(vmhip_mesh* M, const vmhip_tree_element* elements, int32_t n_elements) {
    static_assert(sizeof(vmhip_tree_element) == sizeof(VmTreeElement), "the tree is uploaded as it comes");
    if (!M || !elements || n_elements <= 0) return fail(VMHIP_ERR_ARGUMENT, "mesh_attach_tree: bad arguments");
    for (int32_t i = 0; i < n_elements; ++i) {
        const vmhip_tree_element& e = elements[i];
        const bool leaf = e.child[0] < 0;
        if (e.first < 0 || e.last < e.first || e.last > M->n_nodes || (leaf ? e.child[1] >= 0 : (e.child[0] >= n_elements || e.child[1] < 0 || e.child[1] >= n_elements)))
            return fail(VMHIP_ERR_ARGUMENT, "mesh_attach_tree: an element points outside the mesh or the tree");
        /* children come after their parent (the walk's lists hold every element at most once) */
        if (!leaf && (e.child[0] <= i || e.child[1] <= i)) return fail(VMHIP_ERR_ARGUMENT, "mesh_attach_tree: children must follow their parent");
    }
    if (M->d_tree) (void) hipFree(M->d_tree);
    M->d_tree = nullptr, M->n_elements = 0;
    const size_t bytes = sizeof(VmTreeElement) * size_t(n_elements);
    if (hipMalloc(&M->d_tree, bytes) != hipSuccess || hipMemcpy(M->d_tree, elements, bytes, hipMemcpyHostToDevice) != hipSuccess) {
        if (M->d_tree) (void) hipFree(M->d_tree);
        M->d_tree = nullptr;
        return fail(VMHIP_ERR_HIP, "mesh_attach_tree: device allocation or copy failed");
    }
    M->n_elements = n_elements;
    return VMHIP_OK;
}

int vmhip_batch_create(vmhip_engine* E, vmhip_batch** out) {
    if (!E || !out) return fail(VMHIP_ERR_ARGUMENT, "batch_create: null argument");
    *out = new vmhip_batch();
    (*out)->engine = E;
    return VMHIP_OK;
}
void vmhip_batch_destroy(vmhip_batch* b) {
    if (!b) return;
    if (b->engine && b->engine->stream) (void) hipStreamSynchronize(b->engine->stream);
    b->release();
    delete b;
}
/* Runs the lookup of every frame that asks for it on the device and returns the frames with their ranges filled in
 * (in `patched`, whose range pointers point into b->device_ranges). */
static int lookup_on_device(vmhip_batch* b, const vmhip_frame* frames, int32_t n_frames, std::vector<vmhip_frame>& patched) {
    vmhip_engine* E = b->engine;
    hipStream_t s = E->stream;
    patched.assign(frames, frames + n_frames);
    std::vector<int> who;
    for (int f = 0; f < n_frames; ++f)
        if (frames[f].lookup) who.push_back(f);
    b->device_ranges.assign(n_frames, std::vector<int32_t>());
    if (who.empty()) return VMHIP_OK;
    const int n = int(who.size());
    /* workspace: the frame table, then per frame its bit map and two lists, then the cursor, the verdicts and the
     * dense output */
    size_t bytes = align_up(sizeof(VmLookupFrame) * n, 256);
    std::vector<size_t> at_covered(n), at_list(n);
    size_t dense_words = 0;
    for (int i = 0; i < n; ++i) {
        const vmhip_frame& in = frames[who[i]];
        if (!in.mesh || !in.mesh->d_tree) return fail(VMHIP_ERR_ARGUMENT, "stage: a frame asks for the lookup on the device but its mesh has no tree");
        if (in.lens.projection < VMHIP_RECTILINEAR || in.lens.projection > VMHIP_EQUIDISTANT)
            return fail(VMHIP_ERR_LENS, "Cannot project: Unknown lens type");
        at_covered[i] = bytes;
        bytes += align_up(4 * ((size_t(in.mesh->n_nodes) + 31) / 32), 256);
        at_list[i] = bytes;
        bytes += 2 * align_up(4 * size_t(in.mesh->n_elements), 256);
        dense_words += 2 * size_t(in.mesh->n_elements) + 1;
    }
    const size_t at_cursor = bytes;
    bytes += 256;
    const size_t at_verdict = bytes;
    bytes += align_up(12 * size_t(n), 256);
    const size_t at_dense = bytes;
    bytes += 4 * dense_words;
    HIP_TRY(b->d_lookup_ws.reserve(bytes));
    char* const ws = static_cast<char*>(b->d_lookup_ws.p);
    std::vector<VmLookupFrame> table(n);
    for (int i = 0; i < n; ++i) {
        const vmhip_frame& in = frames[who[i]];
        VmLookupFrame& L = table[i];
        std::memset(&L, 0, sizeof(L));
        VmFrame& d = L.frame;
        d.rays = in.mesh->d_rays;
        d.n_nodes = in.mesh->n_nodes;
        std::memcpy(d.Rco, in.Rco, sizeof(d.Rco));
        d.focal = in.lens.focal_length;
        d.centre_x = in.lens.centre[0];
        d.centre_y = in.lens.centre[1];
        vm_host_inverse_coefficients(in.lens.k, d.ik);
        d.width = in.lens.width;
        d.height = in.lens.height;
        d.projection = in.lens.projection;
        L.tree = in.mesh->d_tree;
        L.n_elements = in.mesh->n_elements;
        L.cos_half_fov = in.lookup->cos_half_fov;
        L.sin_half_fov = in.lookup->sin_half_fov;
        std::memcpy(L.edge, in.lookup->edge, sizeof(L.edge));
        L.covered = reinterpret_cast<uint32_t*>(ws + at_covered[i]);
        L.list[0] = reinterpret_cast<int32_t*>(ws + at_list[i]);
        L.list[1] = reinterpret_cast<int32_t*>(ws + at_list[i] + align_up(4 * size_t(in.mesh->n_elements), 256));
        L.capacity = in.mesh->n_elements;
        L.cursor = reinterpret_cast<int32_t*>(ws + at_cursor);
        L.dense = reinterpret_cast<int32_t*>(ws + at_dense);
        L.verdict = reinterpret_cast<int32_t*>(ws + at_verdict) + 3 * i;
    }
    HIP_TRY(hipMemsetAsync(ws + at_cursor, 0, 4, s));
    HIP_TRY(hipMemcpyAsync(ws, table.data(), sizeof(VmLookupFrame) * n, hipMemcpyHostToDevice, s));
    vm_launch_lookup(reinterpret_cast<const VmLookupFrame*>(ws), n, s);
    HIP_TRY(hipGetLastError());
    std::vector<int32_t> verdict(3 * size_t(n));
    HIP_TRY(hipMemcpyAsync(verdict.data(), ws + at_verdict, 12 * size_t(n), hipMemcpyDeviceToHost, s));
    HIP_TRY(hipStreamSynchronize(s));
    size_t used = 0;
    for (int i = 0; i < n; ++i) {
        if (verdict[3 * i] < 0) return fail(VMHIP_ERR_CAPACITY, "stage: a lookup on the device produced more ranges than it has room for");
        used = std::max(used, size_t(verdict[3 * i + 2]) + 2 * size_t(verdict[3 * i]) + 1);
    }
    std::vector<int32_t> dense(std::max<size_t>(used, 1));
    HIP_TRY(hipMemcpy(dense.data(), ws + at_dense, 4 * used, hipMemcpyDeviceToHost));
    for (int i = 0; i < n; ++i) {
        const int f = who[i], runs = verdict[3 * i];
        const int32_t* first = dense.data() + verdict[3 * i + 2];
        const int32_t* prefix = first + runs;
        std::vector<int32_t>& r = b->device_ranges[f];
        r.resize(2 * size_t(runs));
        for (int k = 0; k < runs; ++k) {
            r[2 * k] = first[k];
            r[2 * k + 1] = first[k] + (prefix[k + 1] - prefix[k]);
        }
        patched[f].ranges = r.data();
        patched[f].n_ranges = runs;
    }
    return VMHIP_OK;
}

static int stage_entry(vmhip_batch* b, const vmhip_frame* frames, int32_t n_frames, int32_t classify, bool wait) {
    if (!b) return fail(VMHIP_ERR_ARGUMENT, "batch_stage: null batch");
    if (b->in_flight) return fail(VMHIP_ERR_ARGUMENT, "batch_stage: a run of this batch is still in flight (vmhip_batch_wait first)");
    if (b->fetching) return fail(VMHIP_ERR_ARGUMENT, "batch_stage: a fetch of this batch is still in flight (vmhip_batch_fetch_wait first)");
    if (!frames || n_frames <= 0) return fail(VMHIP_ERR_ARGUMENT, "stage: no frames");
    std::vector<vmhip_frame> patched;
    int rc = lookup_on_device(b, frames, n_frames, patched);
    if (rc == VMHIP_OK) rc = batch_stage(b, patched.data(), n_frames, classify, wait);
    if (rc != VMHIP_OK) b->frames.clear();
    return rc;
}
int vmhip_batch_stage(vmhip_batch* b, const vmhip_frame* frames, int32_t n_frames, int32_t classify) {
    return stage_entry(b, frames, n_frames, classify, true);
}
int vmhip_batch_stage_async(vmhip_batch* b, const vmhip_frame* frames, int32_t n_frames, int32_t classify) {
    return stage_entry(b, frames, n_frames, classify, false);
}
int vmhip_batch_run(vmhip_batch* b) {
    if (!b) return fail(VMHIP_ERR_ARGUMENT, "batch_run: null batch");
    return batch_run(b);
}
int vmhip_batch_ranges(const vmhip_batch* b, int32_t frame, int32_t* ranges, int32_t capacity) {
    if (!b || frame < 0 || frame >= int32_t(b->frames.size())) return fail(VMHIP_ERR_ARGUMENT, "batch_ranges: no such staged frame");
    const HostFrame& hf = b->frames[frame];
    const int32_t n = int32_t(hf.first.size());
    if (ranges) {
        if (capacity < n) return fail(VMHIP_ERR_CAPACITY, "batch_ranges: more ranges than the array holds");
        for (int32_t r = 0; r < n; ++r) {
            ranges[2 * r] = hf.first[r];
            ranges[2 * r + 1] = hf.first[r] + (hf.prefix[r + 1] - hf.prefix[r]);
        }
    }
    return n;
}
int vmhip_batch_export(vmhip_batch* b, int32_t edge_type, vmhip_lookup_export* per_frame) {
    if (!b || !per_frame) return fail(VMHIP_ERR_ARGUMENT, "batch_export: null argument");
    if (b->frames.empty()) return fail(VMHIP_ERR_ARGUMENT, "batch_export: nothing staged");
    if (b->in_flight) return fail(VMHIP_ERR_ARGUMENT, "batch_export: a run of this batch is still in flight (vmhip_batch_wait first)");
    if (b->fetching) return fail(VMHIP_ERR_ARGUMENT, "batch_export: a fetch of this batch is still in flight (vmhip_batch_fetch_wait first)");
    if (edge_type != VMHIP_EDGE_HARD && edge_type != VMHIP_EDGE_SAME) return fail(VMHIP_ERR_ARGUMENT, "batch_export: unknown edge type");
    const int n = int(b->frames.size());
    for (int f = 0; f < n; ++f) per_frame[f].n_points = b->frames[f].dev.n_cand; /* all of them, so that a caller can size */
    for (int f = 0; f < n; ++f) {
        if (per_frame[f].capacity < per_frame[f].n_points) return fail(VMHIP_ERR_CAPACITY, "batch_export: capacity is smaller than the number of nodes in the frame's ranges");
        if (per_frame[f].n_points > 0 && (!per_frame[f].vectors || !per_frame[f].graph)) return fail(VMHIP_ERR_ARGUMENT, "batch_export: null output array");
    }
    hipStream_t s = b->engine->stream;
    const size_t slots = std::max<size_t>(b->cand_total, 1), width = size_t(b->dev.nb_stride) + 1;
    const size_t at_graph = align_up(12 * slots, 256), at_pixels = at_graph + align_up(4 * slots * width, 256);
    HIP_TRY(b->d_export.reserve(at_pixels + 8 * slots));
    char* const ws = static_cast<char*>(b->d_export.p);
    float* const vectors = reinterpret_cast<float*>(ws);
    int32_t* const graph = reinterpret_cast<int32_t*>(ws + at_graph);
    float* const pixels = reinterpret_cast<float*>(ws + at_pixels);
    vm_launch_lookup_export(b->dev_exact(), edge_type == VMHIP_EDGE_SAME, vectors, graph, pixels, s);
    HIP_TRY(hipGetLastError());
    for (int f = 0; f < n; ++f) {
        const VmFrame& d = b->frames[f].dev;
        const size_t base = size_t(d.cand_base), count = size_t(d.n_cand);
        if (count == 0) continue;
        HIP_TRY(hipMemcpyAsync(per_frame[f].vectors, vectors + base * 3, 12 * count, hipMemcpyDeviceToHost, s));
        HIP_TRY(hipMemcpyAsync(per_frame[f].graph, graph + base * width, 4 * count * size_t(d.nn + 1), hipMemcpyDeviceToHost, s));
        if (per_frame[f].pixels) HIP_TRY(hipMemcpyAsync(per_frame[f].pixels, pixels + base * 2, 8 * count, hipMemcpyDeviceToHost, s));
    }
    HIP_TRY(hipStreamSynchronize(s));
    return VMHIP_OK;
}
int vmhip_batch_run_async(vmhip_batch* b) {
    if (!b) return fail(VMHIP_ERR_ARGUMENT, "batch_run_async: null batch");
    if (b->frames.empty()) return fail(VMHIP_ERR_ARGUMENT, "run: nothing staged");
    if (b->in_flight) return fail(VMHIP_ERR_ARGUMENT, "run: a run of this batch is still in flight (vmhip_batch_wait first)");
    if (b->fetching) return fail(VMHIP_ERR_ARGUMENT, "run: a fetch of this batch is still in flight (vmhip_batch_fetch_wait first)");
    b->have_run = false;
    const int rc = batch_launch(b);
    if (rc == VMHIP_OK) b->in_flight = true;
    return rc;
}
int vmhip_batch_wait(vmhip_batch* b) {
    if (!b) return fail(VMHIP_ERR_ARGUMENT, "batch_wait: null batch");
    if (!b->in_flight) return fail(VMHIP_ERR_ARGUMENT, "batch_wait: no run in flight");
    b->in_flight = false;
    return batch_complete(b);
}
int vmhip_batch_graph_stats(const vmhip_batch* b, int64_t* captures, int64_t* graph_launches, int64_t* eager_launches) {
    if (!b) return fail(VMHIP_ERR_ARGUMENT, "batch_graph_stats: null batch");
    if (captures) *captures = b->graph_captures;
    if (graph_launches) *graph_launches = b->graph_launches;
    if (eager_launches) *eager_launches = b->eager_launches;
    return VMHIP_OK;
}
int vmhip_batch_counts(const vmhip_batch* b, int32_t* n_visible) {
    if (!b || !n_visible || !b->have_run) return fail(VMHIP_ERR_ARGUMENT, "batch_counts: no completed run");
    std::copy(b->h_V.begin(), b->h_V.end(), n_visible);
    return VMHIP_OK;
}
int vmhip_batch_fetch(vmhip_batch* b, vmhip_result* results) {
    if (!b) return fail(VMHIP_ERR_ARGUMENT, "batch_fetch: null batch");
    return batch_fetch(b, results);
}
int vmhip_batch_fetch_async(vmhip_batch* b, vmhip_result* results) {
    if (!b) return fail(VMHIP_ERR_ARGUMENT, "batch_fetch_async: null batch");
    const int rc = batch_fetch_enqueue(b, results);
    if (rc != VMHIP_OK) {
        (void) hipStreamSynchronize(b->engine->stream); /* copies queued before the failure write into the caller's arrays */
        return rc;
    }
    b->fetching = true;
    return VMHIP_OK;
}
size_t vmhip_batch_fetch_packed_size(const vmhip_batch* b) {
    if (!b || !b->have_run) return 0;
    return packed_layout(b, nullptr);
}
int vmhip_batch_fetch_packed_async(vmhip_batch* b, void* block, size_t bytes, vmhip_result* results) {
    if (!b) return fail(VMHIP_ERR_ARGUMENT, "batch_fetch_packed_async: null batch");
    const int rc = batch_fetch_packed_enqueue(b, block, bytes, results);
    if (rc != VMHIP_OK) {
        (void) hipStreamSynchronize(b->engine->stream);
        return rc;
    }
    b->fetching = true;
    return VMHIP_OK;
}
int vmhip_batch_fetch_wait(vmhip_batch* b) {
    if (!b) return fail(VMHIP_ERR_ARGUMENT, "batch_fetch_wait: null batch");
    if (!b->fetching) return fail(VMHIP_ERR_ARGUMENT, "batch_fetch_wait: no fetch in flight");
    b->fetching = false;
    HIP_TRY(hipStreamSynchronize(b->engine->stream));
    return VMHIP_OK;
}
void* vmhip_host_alloc(size_t bytes) {
    void* p = nullptr;
    if (hipHostMalloc(&p, bytes ? bytes : 1, hipHostMallocDefault) != hipSuccess) {
        (void) hipGetLastError();
        return nullptr;
    }
    return p;
}
void vmhip_host_free(void* memory) {
    if (memory) (void) hipHostFree(memory);
}

int vmhip_batch_detect(vmhip_batch* b, int32_t class_index, float threshold, int32_t arg_max_only, int32_t clusters,
                       vmhip_detections* out) {
    if (!b || !out) return fail(VMHIP_ERR_ARGUMENT, "batch_detect: null argument");
    if (!b->have_run || !b->classify || !b->final_act) return fail(VMHIP_ERR_ARGUMENT, "batch_detect: no completed classifying run");
    if (b->fetching) return fail(VMHIP_ERR_ARGUMENT, "batch_detect: a fetch of this batch is still in flight (vmhip_batch_fetch_wait first)");
    vmhip_engine* E = b->engine;
    const int C = E->n_classes;
    if (class_index < 0 || class_index >= C) return fail(VMHIP_ERR_ARGUMENT, "batch_detect: no such class");
    const int n = int(b->frames.size());
    hipStream_t s = E->stream;
    HIP_TRY(b->d_detect.reserve(vm_detect_workspace_bytes(b->row_total, n)));
    VmDetectDev D{};
    vm_detect_carve(b->d_detect.p, b->row_total, n, &D);
    D.probabilities = b->final_act;
    D.n_classes = C, D.class_index = class_index, D.arg_max_only = arg_max_only != 0, D.threshold = threshold;
    /* a caller that was told its arrays are too small asks again with the same arguments: nothing to recompute */
    const bool held = !b->d_detect.grew && b->detect_serial == b->run_serial && b->detect_class == class_index
                      && std::memcmp(&b->detect_threshold, &threshold, sizeof(float)) == 0 && b->detect_arg_max == (arg_max_only != 0)
                      && b->detect_clusters == (clusters != 0);
    if (!held) {
        vm_launch_detect(b->dev_exact(), D, clusters != 0, s);
        HIP_TRY(hipGetLastError());
        b->detect_serial = b->run_serial, b->detect_class = class_index, b->detect_threshold = threshold;
        b->detect_arg_max = arg_max_only != 0, b->detect_clusters = clusters != 0;
    }
    /* counts first (pinned, one wait), then one dense block with everything, then it is a matter of host copies */
    auto pinned = [&](size_t bytes) -> hipError_t {
        if (bytes <= b->h_detect_cap) return hipSuccess;
        if (b->h_detect) (void) hipHostFree(b->h_detect);
        b->h_detect = nullptr, b->h_detect_cap = 0;
        hipError_t e = hipHostMalloc(&b->h_detect, bytes + bytes / 4 + 4096, hipHostMallocDefault);
        if (e == hipSuccess) b->h_detect_cap = bytes + bytes / 4 + 4096;
        return e;
    };
    HIP_TRY(pinned(size_t(n) * 8));
    int32_t* counts = static_cast<int32_t*>(b->h_detect);
    HIP_TRY(hipMemcpyAsync(counts, D.counts, size_t(n) * 8, hipMemcpyDeviceToHost, s));
    HIP_TRY(hipStreamSynchronize(s));
    bool fits = true;
    size_t total_d = 0, total_c = 0;
    std::vector<int32_t> nd(n), nc(n);
    for (int f = 0; f < n; ++f) {
        nd[f] = counts[2 * f], nc[f] = clusters ? counts[2 * f + 1] : 0;
        out[f].n_detections = nd[f];
        out[f].n_clusters = nc[f];
        total_d += size_t(nd[f]), total_c += size_t(nc[f]);
        fits = fits && out[f].capacity >= nd[f] && (!clusters || out[f].cluster_capacity >= nc[f]);
    }
    if (!fits) return fail(VMHIP_ERR_CAPACITY, "batch_detect: a frame has more detections or clusters than its arrays hold");
    if (total_d == 0) return VMHIP_OK;
    if (total_d > 0x7fffffffull) return fail(VMHIP_ERR_CAPACITY, "batch_detect: too many detections for one download");
    const size_t words = 5 * total_d + 7 * total_c;
    HIP_TRY(b->d_detect_packed.reserve(words * 4));
    HIP_TRY(pinned(words * 4));
    vm_launch_detect_pack(b->dev_exact(), D, static_cast<uint32_t*>(b->d_detect_packed.p), int(total_d), int(total_c), s);
    HIP_TRY(hipGetLastError());
    HIP_TRY(hipMemcpyAsync(b->h_detect, b->d_detect_packed.p, words * 4, hipMemcpyDeviceToHost, s));
    HIP_TRY(hipStreamSynchronize(s));
    const uint32_t* node = static_cast<const uint32_t*>(b->h_detect);
    const uint32_t* pixel = node + total_d;
    const uint32_t* probability = pixel + 2 * total_d;
    const uint32_t* cluster = probability + total_d;
    const uint32_t* size = cluster + total_d;
    const uint32_t* box = size + total_c;
    const uint32_t* sum = box + 4 * total_c;
    size_t d0 = 0, c0 = 0;
    for (int f = 0; f < n; ++f) {
        vmhip_detections& R = out[f];
        const size_t d = size_t(nd[f]), c = size_t(nc[f]);
        if (R.node) std::memcpy(R.node, node + d0, 4 * d);
        if (R.pixel) std::memcpy(R.pixel, pixel + 2 * d0, 8 * d);
        if (R.probability) std::memcpy(R.probability, probability + d0, 4 * d);
        if (R.cluster && clusters) std::memcpy(R.cluster, cluster + d0, 4 * d);
        if (R.cluster_size) std::memcpy(R.cluster_size, size + c0, 4 * c);
        if (R.cluster_box) std::memcpy(R.cluster_box, box + 4 * c0, 16 * c);
        if (R.cluster_centre) {
            const float* sums = reinterpret_cast<const float*>(sum + 2 * c0);
            for (size_t k = 0; k < c; ++k) {
                R.cluster_centre[2 * k] = sums[2 * k] / float(int32_t(size[c0 + k]));
                R.cluster_centre[2 * k + 1] = sums[2 * k + 1] / float(int32_t(size[c0 + k]));
            }
        }
        d0 += d, c0 += c;
    }
    return VMHIP_OK;
}

int vmhip_batch_profile(vmhip_batch* b, int32_t enable) {
    if (!b) return fail(VMHIP_ERR_ARGUMENT, "batch_profile: null batch");
    if (enable < 0 || enable > 2) return fail(VMHIP_ERR_ARGUMENT, "batch_profile: mode must be 0, 1 or 2");
    if (enable == 2) {
        if (b->profile != 1 || !b->have_run) return fail(VMHIP_ERR_ARGUMENT, "batch_profile: mode 2 follows a run profiled in mode 1");
        std::map<std::string, float> total;
        for (int i = 0; i < b->n_slots; ++i) {
            float ms = 0.0f;
            HIP_TRY(hipEventElapsedTime(&ms, b->events[2 * i], b->events[2 * i + 1]));
            total[b->slot_names[i]] += ms;
        }
        std::string longest;
        float best = -1.0f;
        for (const auto& kv : total)
            if (kv.second > best) best = kv.second, longest = kv.first;
        b->slot_wanted.assign(b->n_slots, 0);
        for (int i = 0; i < b->n_slots; ++i) b->slot_wanted[i] = longest == b->slot_names[i];
    }
    if (b->profile != enable) b->drop_graph(); /* a captured run holds the event records of its mode, or none */
    b->profile = enable;
    return VMHIP_OK;
}
int vmhip_batch_profile_read(vmhip_batch* b, int32_t max_slots, int32_t* n_slots, const char** names, float* milliseconds,
                             int64_t* units) {
    if (!b || !n_slots) return fail(VMHIP_ERR_ARGUMENT, "batch_profile_read: null argument");
    if (!b->profile || !b->have_run) return fail(VMHIP_ERR_ARGUMENT, "batch_profile_read: profiling was not enabled for the last run");
    int n = 0;
    for (int i = 0; i < b->n_slots && n < max_slots; ++i) {
        if (b->profile == 2 && !b->slot_wanted[i]) continue;
        float ms = 0.0f;
        HIP_TRY(hipEventElapsedTime(&ms, b->events[2 * i], b->events[2 * i + 1]));
        if (names) names[n] = b->slot_names[i];
        if (milliseconds) milliseconds[n] = ms;
        if (units) units[n] = b->slot_units[i];
        ++n;
    }
    *n_slots = n;
    return VMHIP_OK;
}

int vmhip_debug_set(int32_t what, double value) {
    switch (what) {
        case VMHIP_DEBUG_FLOW_POLL_LIMIT: {
            const int polls = value <= 0.0 ? VM_FLOW_POLL_LIMIT_DEFAULT : int(value);
            HIP_TRY(vm_flow_set_poll_limit(polls));
            return VMHIP_OK;
        }
        case VMHIP_DEBUG_PROJECTION_ERROR: g_debug_px_error.store(float(value)); return VMHIP_OK;
        case VMHIP_DEBUG_WIDE_OFFSETS: g_debug_wide_offsets.store(value != 0.0); return VMHIP_OK;
        case VMHIP_DEBUG_STAMP_ROW_BITS: g_debug_stamp_row_bits.store(int(value)); return VMHIP_OK;
        case VMHIP_DEBUG_EDGE_BAND: g_debug_edge_band.store(value <= 0.0 ? VMHIP_AMB_EPS_DEFAULT : float(value)); return VMHIP_OK;
        default: return fail(VMHIP_ERR_ARGUMENT, "debug_set: unknown knob");
    }
}
int vmhip_batch_guard_stats(const vmhip_batch* b, int64_t* listed, int64_t* most_listed, int64_t* overruled, int64_t* reruns) {
    if (!b) return fail(VMHIP_ERR_ARGUMENT, "batch_guard_stats: null batch");
    if (listed) *listed = b->amb_seen;
    if (most_listed) *most_listed = b->amb_most;
    if (overruled) *overruled = b->overruled;
    if (reruns) *reruns = b->reruns;
    return VMHIP_OK;
}

int vmhip_selftest_libm(int32_t which, const float* x, float* y, int32_t n) {
    if (!x || !y || n <= 0 || which < 0 || which > 3) return fail(VMHIP_ERR_ARGUMENT, "selftest_libm: bad arguments");
    float *dx = nullptr, *dy = nullptr;
    HIP_TRY(hipMalloc(&dx, 4 * size_t(n)));
    if (hipMalloc(&dy, 4 * size_t(n)) != hipSuccess) {
        (void) hipFree(dx);
        return fail(VMHIP_ERR_HIP, "selftest_libm: out of device memory");
    }
    hipError_t e = hipMemcpy(dx, x, 4 * size_t(n), hipMemcpyHostToDevice);
    if (e == hipSuccess) {
        vm_launch_libm(which, dx, dy, n, nullptr);
        e = hipMemcpy(y, dy, 4 * size_t(n), hipMemcpyDeviceToHost);
    }
    (void) hipFree(dx);
    (void) hipFree(dy);
    if (e != hipSuccess) return fail(VMHIP_ERR_HIP, std::string("selftest_libm: ") + hipGetErrorString(e));
    return VMHIP_OK;
}

int vmhip_selftest_copy(int64_t bytes, int32_t repeats, float* ms) {
    if (bytes <= 0 || bytes % 16 != 0 || repeats <= 0) return fail(VMHIP_ERR_ARGUMENT, "selftest_copy: bad arguments");
    void *src = nullptr, *dst = nullptr;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    hipError_t e = hipMalloc(&src, size_t(bytes));
    if (e == hipSuccess) e = hipMalloc(&dst, size_t(bytes));
    if (e == hipSuccess) e = hipMemset(src, 1, size_t(bytes));
    if (e == hipSuccess) e = hipEventCreate(&e0);
    if (e == hipSuccess) e = hipEventCreate(&e1);
    if (e == hipSuccess) {
        vm_launch_copy_probe(src, dst, size_t(bytes), nullptr); /* warm-up */
        e = hipEventRecord(e0, nullptr);
        for (int i = 0; i < repeats && e == hipSuccess; ++i) vm_launch_copy_probe(src, dst, size_t(bytes), nullptr);
        if (e == hipSuccess) e = hipEventRecord(e1, nullptr);
        if (e == hipSuccess) e = hipEventSynchronize(e1);
        float total = 0.0f;
        if (e == hipSuccess) e = hipEventElapsedTime(&total, e0, e1);
        if (ms) *ms = total / float(repeats);
    }
    if (e0) (void) hipEventDestroy(e0);
    if (e1) (void) hipEventDestroy(e1);
    if (src) (void) hipFree(src);
    if (dst) (void) hipFree(dst);
    if (e != hipSuccess) return fail(VMHIP_ERR_HIP, std::string("selftest_copy: ") + hipGetErrorString(e));
    return VMHIP_OK;
}

int vmhip_selftest_stream(int64_t rows, int32_t read_bytes_per_row, int32_t write_bytes_per_row, int32_t repeats, float* ms) {
    if (rows <= 0 || rows % 64 != 0 || read_bytes_per_row <= 0 || read_bytes_per_row % 4 != 0 || write_bytes_per_row <= 0 || write_bytes_per_row % 4 != 0
        || repeats <= 0)
        return fail(VMHIP_ERR_ARGUMENT, "selftest_stream: bad arguments");
    void *src = nullptr, *dst = nullptr;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    const size_t rd = size_t(rows) * read_bytes_per_row, wr = size_t(rows) * write_bytes_per_row;
    hipError_t e = hipMalloc(&src, rd);
    if (e == hipSuccess) e = hipMalloc(&dst, wr);
    if (e == hipSuccess) e = hipMemset(src, 1, rd);
    if (e == hipSuccess) e = hipEventCreate(&e0);
    if (e == hipSuccess) e = hipEventCreate(&e1);
    if (e == hipSuccess) {
        vm_launch_stream_probe(src, dst, size_t(rows), read_bytes_per_row, write_bytes_per_row, nullptr); /* warm-up */
        e = hipEventRecord(e0, nullptr);
        for (int i = 0; i < repeats && e == hipSuccess; ++i) vm_launch_stream_probe(src, dst, size_t(rows), read_bytes_per_row, write_bytes_per_row, nullptr);
        if (e == hipSuccess) e = hipEventRecord(e1, nullptr);
        if (e == hipSuccess) e = hipEventSynchronize(e1);
        float total = 0.0f;
        if (e == hipSuccess) e = hipEventElapsedTime(&total, e0, e1);
        if (ms) *ms = total / float(repeats);
    }
    if (e0) (void) hipEventDestroy(e0);
    if (e1) (void) hipEventDestroy(e1);
    if (src) (void) hipFree(src);
    if (dst) (void) hipFree(dst);
    if (e != hipSuccess) return fail(VMHIP_ERR_HIP, std::string("selftest_stream: ") + hipGetErrorString(e));
    return VMHIP_OK;
}

int vmhip_classify_batch(vmhip_engine* E, const vmhip_frame* frames, int32_t n_frames, vmhip_result* results) {
    if (!E) return fail(VMHIP_ERR_ARGUMENT, "classify_batch: null engine");
    ensure_scratch(E);
    int rc = vmhip_batch_stage(E->scratch, frames, n_frames, 1);
    if (rc == VMHIP_OK) rc = batch_run(E->scratch);
    if (rc == VMHIP_OK) rc = batch_fetch(E->scratch, results);
    return rc;
}
int vmhip_classify(vmhip_engine* E, const vmhip_frame* frame, vmhip_result* result) {
    return vmhip_classify_batch(E, frame, 1, result);
}
int vmhip_project(vmhip_engine* E, const vmhip_frame* frame, vmhip_result* result) {
    if (!E) return fail(VMHIP_ERR_ARGUMENT, "project: null engine");
    ensure_scratch(E);
    int rc = vmhip_batch_stage(E->scratch, frame, 1, 0);
    if (rc == VMHIP_OK) rc = batch_run(E->scratch);
    if (rc == VMHIP_OK) rc = batch_fetch(E->scratch, result);
    return rc;
}
}

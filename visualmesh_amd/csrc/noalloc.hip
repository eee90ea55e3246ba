/*
 * noalloc.hip - vmhip_project_noalloc: the projection of one frame (candidate projection, on-screen filter,
 * order-preserving compaction, neighbourhood table) as a sequence of kernel launches and nothing else. No hipMalloc,
 * no hipFree, no copy, no wait: usable on a stream that is being captured into a HIP graph and from loops that must
 * not allocate. The kernels are those of vmhip_project (project.hip); what vmhip_project keeps in a workspace that
 * grows with the batch lives here in one array of fixed size inside the library's device image.
 *
 * The array exists once per device and keeps its contents between calls: the reverse lookup table is validated by a
 * run stamp that the first kernel of every call advances (so it is never cleared, except when the 8-bit stamp starts
 * again after 255 calls, which a kernel of every call checks for), everything else is rewritten by the call before it is read. Calls that
 * overlap on one device race on the array.
 */
#include <atomic>
#include <mutex>

#include "vmhip_internal.h"

namespace {

constexpr size_t up256(size_t v) { return (v + 255) / 256 * 256; }

constexpr size_t MAX_CAND = VMHIP_NOALLOC_MAX_CANDIDATES;
constexpr size_t MAX_NODES = VMHIP_NOALLOC_MAX_NODES;
constexpr size_t MAX_RANGES = VMHIP_NOALLOC_MAX_RANGES;
static_assert(MAX_CAND % VMHIP_TILE == 0, "whole candidate tiles");

/* layout of the array, every part on a 256-byte boundary */
struct Header {
    uint32_t epoch;      /* run stamp of the reverse lookup */
    uint32_t wrapped;    /* the stamp wrapped in this call: the table is cleared before it is stamped again */
    int32_t amb_count;   /* candidates within the edge band (counted by the projection, not used by this entry point) */
};
constexpr size_t AT_HEADER = 0;
constexpr size_t AT_FRAME = AT_HEADER + 256;
constexpr size_t AT_RANGE_FIRST = AT_FRAME + up256(sizeof(VmFrame));
constexpr size_t AT_RANGE_PREFIX = AT_RANGE_FIRST + up256(4 * MAX_RANGES);
constexpr size_t AT_CAND_PX = AT_RANGE_PREFIX + up256(4 * (MAX_RANGES + 1));
constexpr size_t AT_CAND_G = AT_CAND_PX + up256(8 * MAX_CAND);
constexpr size_t AT_CAND_KEEP = AT_CAND_G + up256(4 * MAX_CAND);
constexpr size_t AT_TILE_COUNT = AT_CAND_KEEP + up256(MAX_CAND / 8);
constexpr size_t AT_NO_FORCE = AT_TILE_COUNT + up256(4 * (MAX_CAND / VMHIP_TILE)); /* stays zero: no forced decisions */
constexpr size_t AT_AMB_LIST = AT_NO_FORCE + up256(MAX_CAND / 8);
constexpr size_t AT_LOOKUP = AT_AMB_LIST + up256(sizeof(int2) * VMHIP_AMB_CAP);
constexpr size_t SCRATCH_BYTES = AT_LOOKUP + up256(sizeof(uint32_t) * (MAX_NODES + 1));

/* a reverse-lookup entry: 8 bits of run stamp above 24 bits of row */
constexpr int STAMP_ROW_BITS = 24;
constexpr uint32_t STAMP_LAST = 0xffffffffu >> STAMP_ROW_BITS;
static_assert(MAX_CAND < (size_t(1) << STAMP_ROW_BITS), "a row fits the entry");

}  // namespace

/* The workspace of vmhip_project_noalloc, 11.3 MB, held by every device the library runs on until the process ends.
 * In host code this name is a handle, not an address: the address on a device comes from hipGetSymbolAddress
 * (vm_noalloc_setup) and is what every launch below is given. */
static __device__ __align__(256) unsigned char scratch[SCRATCH_BYTES];

namespace {

constexpr int MAX_DEVICES = 64;
std::mutex g_setup_lock;
std::atomic<unsigned char*> g_scratch_ptr[MAX_DEVICES];

constexpr int PREPARE_THREADS = 1024;

/* First kernel of a call, one block: advances the run stamp, turns the caller's (first, one-past-last) pairs into the
 * range table the projection reads (first[r], exclusive prefix of the lengths), checks the pairs (ascending, disjoint,
 * inside the mesh, lengths summing to the candidate count the grids were sized for) and writes the frame descriptor.
 * A rejected table leaves a frame without candidates and -1 in *n_visible; the kernels that follow then write nothing. */
__global__ __launch_bounds__(PREPARE_THREADS) void vm_noalloc_prepare_kernel(VmFrame F, const int32_t* __restrict__ ranges, int n_candidates,
                                                                               Header* header, VmFrame* frame_out, int32_t* range_first,
                                                                               int32_t* range_prefix, int32_t* n_visible, int32_t* neighbourhood) {
    __shared__ int wave_total[PREPARE_THREADS / 64];
    __shared__ int bad;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    if (tid == 0) {
        bad = 0;
        const uint32_t e = header->epoch + 1u;
        header->wrapped = e > STAMP_LAST ? 1u : 0u;
        header->epoch = e > STAMP_LAST ? 1u : e;
        header->amb_count = 0;
    }
    __syncthreads();
    long long running = 0; /* candidates in the ranges before this round's */
    for (int base = 0; base < F.n_ranges; base += PREPARE_THREADS) {
        const int r = base + tid;
        int first = 0, length = 0;
        if (r < F.n_ranges) {
            first = ranges[2 * r];
            const int last = ranges[2 * r + 1];
            const int previous_last = r > 0 ? ranges[2 * r - 1] : 0;
            if (first < previous_last || last < first || last > F.n_nodes) atomicOr(&bad, 1);
            else length = last - first;
        }
        int scan = length;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const int up = __shfl_up(scan, d);
            if (lane >= d) scan += up;
        }
        __syncthreads(); /* wave_total of the round before has been read */
        if (lane == 63) wave_total[wave] = scan;
        __syncthreads();
        long long before = running + (scan - length), total = 0;
        for (int w = 0; w < PREPARE_THREADS / 64; ++w) {
            if (w < wave) before += wave_total[w];
            total += wave_total[w];
        }
        if (r < F.n_ranges) {
            range_first[r] = first;
            range_prefix[r] = (int32_t) (before < 0x7fffffffLL ? before : 0x7fffffffLL);
        }
        running += total;
    }
    __syncthreads();
    if (tid == 0) {
        const bool ok = bad == 0 && running == (long long) n_candidates;
        const int n = ok ? n_candidates : 0;
        range_prefix[F.n_ranges] = n;
        F.n_ranges = ok ? F.n_ranges : 0;
        F.n_cand = n;
        F.cand_base = 0, F.cand_tile0 = 0, F.cand_tiles = (n + VMHIP_TILE - 1) / VMHIP_TILE;
        F.row_base = 0, F.row_tile0 = 0, F.row_tiles = n > 0 ? (n + 1 + VMHIP_TILE - 1) / VMHIP_TILE : 0;
        *frame_out = F;
        *n_visible = ok ? 0 : -1;
        /* a frame without candidates has no tile that would write its null row (row 0 then: every neighbour is row 0) */
        if (ok && n == 0)
            for (int j = 0; j < F.nn; ++j) neighbourhood[j] = 0;
    }
}

/* Second kernel of a call: does nothing unless the run stamp started again from one (every 255 calls), then it clears the
 * reverse lookup table so that stamps of 255 calls ago cannot look current. */
__global__ __launch_bounds__(256) void vm_noalloc_wrap_kernel(const Header* header, uint32_t* lookup, size_t entries) {
    if (header->wrapped == 0u) return;
    for (size_t i = (size_t) blockIdx.x * blockDim.x + threadIdx.x; i < entries; i += (size_t) gridDim.x * blockDim.x) lookup[i] = 0u;
}

}  // namespace

hipError_t vm_noalloc_setup(void) {
    int device = 0;
    hipError_t e = hipGetDevice(&device);
    if (e != hipSuccess) return e;
    if (device < 0 || device >= MAX_DEVICES) return hipErrorInvalidDevice;
    if (g_scratch_ptr[device].load(std::memory_order_acquire)) return hipSuccess;
    std::lock_guard<std::mutex> hold(g_setup_lock);
    if (g_scratch_ptr[device].load(std::memory_order_acquire)) return hipSuccess;
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return e;
    if (!p) return hipErrorInvalidSymbol;
    g_scratch_ptr[device].store(static_cast<unsigned char*>(p), std::memory_order_release);
    return hipSuccess;
}

extern "C" int vmhip_project_noalloc(const vmhip_mesh* mesh, const float* Rco, const vmhip_lens* lens, const int32_t* ranges,
                                     int32_t n_ranges, int32_t n_candidates, const vmhip_projection_device* out, void* hip_stream) {
    if (!mesh || !Rco || !lens || !out) return vm_set_error(VMHIP_ERR_ARGUMENT, "project_noalloc: null argument");
    if (lens->projection < VMHIP_RECTILINEAR || lens->projection > VMHIP_EQUIDISTANT)
        return vm_set_error(VMHIP_ERR_LENS, "Cannot project: Unknown lens type");
    if (lens->width <= 0 || lens->height <= 0) return vm_set_error(VMHIP_ERR_ARGUMENT, "project_noalloc: empty image dimensions");
    if (n_ranges < 0 || n_candidates < 0 || (n_ranges > 0 && !ranges)) return vm_set_error(VMHIP_ERR_ARGUMENT, "project_noalloc: bad range table");
    if (size_t(n_ranges) > MAX_RANGES)
        return vm_set_error(VMHIP_ERR_CAPACITY, "project_noalloc: more than VMHIP_NOALLOC_MAX_RANGES (65536) ranges; use vmhip_project");
    if (size_t(n_candidates) > MAX_CAND)
        return vm_set_error(VMHIP_ERR_CAPACITY, "project_noalloc: more than VMHIP_NOALLOC_MAX_CANDIDATES (524288) candidate nodes; use vmhip_project");
    if (size_t(mesh->n_nodes) > MAX_NODES)
        return vm_set_error(VMHIP_ERR_CAPACITY, "project_noalloc: the mesh has more than VMHIP_NOALLOC_MAX_NODES (1048576) nodes; use vmhip_project");
    if (!out->n_visible || !out->pixel_coordinates || !out->global_indices || !out->neighbourhood)
        return vm_set_error(VMHIP_ERR_ARGUMENT, "project_noalloc: null output array");
    if (out->capacity < n_candidates) return vm_set_error(VMHIP_ERR_CAPACITY, "project_noalloc: capacity is smaller than the candidate count");

    int device = 0;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= MAX_DEVICES) return vm_set_error(VMHIP_ERR_HIP, "project_noalloc: no current device");
    if (device != mesh->device) return vm_set_error(VMHIP_ERR_ARGUMENT, "project_noalloc: the mesh lives on another device than the current one");
    unsigned char* ws = g_scratch_ptr[device].load(std::memory_order_acquire);
    if (!ws) { /* every mesh upload has done this for its device; kept for a device handed over some other way */
        if (vm_noalloc_setup() != hipSuccess) return vm_set_error(VMHIP_ERR_HIP, "project_noalloc: the workspace symbol could not be resolved");
        ws = g_scratch_ptr[device].load(std::memory_order_acquire);
    }
    hipStream_t s = static_cast<hipStream_t>(hip_stream);

    Header* header = reinterpret_cast<Header*>(ws + AT_HEADER);
    VmFrame* d_frame = reinterpret_cast<VmFrame*>(ws + AT_FRAME);
    int32_t* range_first = reinterpret_cast<int32_t*>(ws + AT_RANGE_FIRST);
    int32_t* range_prefix = reinterpret_cast<int32_t*>(ws + AT_RANGE_PREFIX);
    uint32_t* lookup = reinterpret_cast<uint32_t*>(ws + AT_LOOKUP);

    VmFrame F{};
    F.rays = mesh->d_rays;
    F.nbr = mesh->d_nbr;
    F.r_lookup = lookup;
    F.n_nodes = mesh->n_nodes;
    F.nn = mesh->nn;
    for (int i = 0; i < 9; ++i) F.Rco[i] = Rco[i];
    F.focal = lens->focal_length;
    F.centre_x = lens->centre[0];
    F.centre_y = lens->centre[1];
    vm_host_inverse_coefficients(lens->k, F.ik);
    F.width = lens->width;
    F.height = lens->height;
    F.projection = lens->projection;
    F.image = nullptr;
    F.fmt = VMHIP_FMT_NONE;
    F.range_first = range_first;
    F.range_prefix = range_prefix;
    F.n_ranges = n_ranges;
    F.force_valid = reinterpret_cast<const uint64_t*>(ws + AT_NO_FORCE);
    F.force_keep = reinterpret_cast<const uint64_t*>(ws + AT_NO_FORCE);

    VmBatchDev B{};
    B.frames = d_frame;
    B.n_frames = 1;
    B.n_cand_tiles = (n_candidates + VMHIP_TILE - 1) / VMHIP_TILE;
    B.n_row_tiles = n_candidates > 0 ? (n_candidates + 1 + VMHIP_TILE - 1) / VMHIP_TILE : 0;
    B.epoch = &header->epoch;
    B.stamp_row_bits = STAMP_ROW_BITS;
    B.uniform_nn = mesh->nn;
    B.wide_offsets = uint64_t(mesh->n_nodes) * uint64_t(mesh->nn) >= (1ull << 30) ? 1 : 0; /* the output tables are far below 4 GiB */
    B.cand_px = reinterpret_cast<float2*>(ws + AT_CAND_PX);
    B.cand_g = reinterpret_cast<int32_t*>(ws + AT_CAND_G);
    B.cand_keep = reinterpret_cast<uint64_t*>(ws + AT_CAND_KEEP);
    B.tile_count = reinterpret_cast<int32_t*>(ws + AT_TILE_COUNT);
    B.frame_V = out->n_visible;
    B.amb_count = &header->amb_count;
    B.amb_list = reinterpret_cast<int2*>(ws + AT_AMB_LIST);
    B.row_px = reinterpret_cast<float2*>(out->pixel_coordinates);
    B.row_gidx = out->global_indices;
    B.row_nb = out->neighbourhood;
    B.nb_stride = mesh->nn;
    B.row_nbl = nullptr, B.tile_halo = nullptr, B.tile_desc = nullptr;
    B.halo_cap = 0;
    B.flow_timeouts = nullptr;
    B.amb_eps = VMHIP_AMB_EPS_DEFAULT;
    B.px_error = 0.0f;

    hipLaunchKernelGGL(vm_noalloc_prepare_kernel, dim3(1), dim3(PREPARE_THREADS), 0, s, F, ranges, n_candidates, header, d_frame, range_first,
                       range_prefix, out->n_visible, out->neighbourhood);
    hipLaunchKernelGGL(vm_noalloc_wrap_kernel, dim3(256), dim3(256), 0, s, header, lookup, size_t(MAX_NODES) + 1);
    vm_launch_project(B, s);
    vm_launch_compact(B, nullptr, 0, s);
    vm_launch_neighbourhood(B, s);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return vm_set_error(VMHIP_ERR_HIP, hipGetErrorString(e));
    return VMHIP_OK;
}

/*
 * detect.hip - what a consumer of the classified mesh does first, done on the device so that only detections cross
 * PCIe: pick the nodes of one class (probability threshold, optionally arg-max only), keep their order, and group
 * them into the connected components of the mesh's neighbourhood graph.
 *
 * The reference has no such step inside its engines: its consumers walk the whole ClassifiedMesh on the host
 * (example/draw.hpp:41-59 colours every node by its classification; the neighbourhood table they would cluster on
 * is the one engine/cpu/engine.hpp:113-129 builds). The kernels here read the results of the last run where they lie:
 * the final activations, the visible nodes' mesh indices and pixels, and the local neighbourhood table.
 *
 *   vm_detect_kernel         one block per frame walks the frame's rows in order: flag, block-wide exclusive scan,
 *                            write the detections densely (order preserving) and a row -> detection map
 *   vm_cluster_union_kernel  one thread per row: a detected row unites itself with every detected neighbour in a
 *                            lock-free union-find (the larger root is hung below the smaller with a compare-and-swap,
 *                            so the smallest detection of a component ends up as its root whatever the order)
 *   vm_cluster_label_kernel  one block per frame: numbers the roots in detection order, labels every detection with
 *                            its root's number and accumulates size, bounding box and pixel sums per cluster
 *   vm_detect_pack_kernel    one block per frame: everything the host wants, densely, for a single download
 */
#include "vmhip_internal.h"

namespace {

constexpr int DETECT_THREADS = 1024;

__device__ __forceinline__ int frame_of_row_tile(const VmFrame* frames, int n, int tile) {
    int lo = 0, hi = n - 1;
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (frames[mid].row_tile0 <= tile) lo = mid;
        else hi = mid - 1;
    }
    return lo;
}

/* exclusive prefix of `flag` over the block, in thread order; total = number of flags set. scratch: one int per wave */
__device__ __forceinline__ int block_rank(bool flag, int* scratch, int& total) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const unsigned long long mask = __ballot(flag);
    const int before = __popcll(mask & ((1ull << lane) - 1ull));
    __syncthreads(); /* scratch may still be read from the previous call */
    if (lane == 0) scratch[wave] = __popcll(mask);
    __syncthreads();
    int offset = 0, sum = 0;
    for (int w = 0; w < DETECT_THREADS / 64; ++w) {
        const int c = scratch[w];
        if (w < wave) offset += c;
        sum += c;
    }
    total = sum;
    return offset + before;
}

__global__ __launch_bounds__(DETECT_THREADS) void vm_detect_kernel(VmBatchDev B, VmDetectDev D) {
    __shared__ int scratch[DETECT_THREADS / 64];
    const int f = blockIdx.x;
    const VmFrame& F = B.frames[f];
    const int V = F.n_cand > 0 ? B.frame_V[f] : 0; /* a frame without candidates has no rows */
    const size_t base = (size_t) F.row_base;
    const int C = D.n_classes, cls = D.class_index;
    int running = 0;
    for (int r0 = 0; r0 < V; r0 += DETECT_THREADS) {
        const int r = r0 + (int) threadIdx.x;
        bool hit = false;
        float p = 0.0f;
        if (r < V) {
            const float* q = D.probabilities + (base + r) * C;
            p = q[cls];
            hit = p >= D.threshold;
            if (hit && D.arg_max_only) { /* the first maximum wins, as std::max_element would have it */
                for (int c = 0; c < C; ++c)
                    if (c < cls ? q[c] >= p : q[c] > p) hit = false;
            }
        }
        int total;
        const int j = running + block_rank(hit, scratch, total);
        if (r < V) D.row_to_detection[base + r] = hit ? j : -1;
        if (hit) {
            D.node[base + j] = B.row_gidx[base + r];
            D.pixel[base + j] = B.row_px[base + r];
            D.probability[base + j] = p;
            D.parent[base + j] = j;
        }
        running += total;
    }
    if (threadIdx.x == 0) {
        if (F.n_cand > 0) D.row_to_detection[base + V] = -1; /* the null row (a frame without candidates owns no row at all) */
        D.counts[2 * f] = running;
        D.counts[2 * f + 1] = 0;
    }
}

/* Parents only ever move to smaller indices (a root is hung below a smaller root, a node is re-pointed at its
 * grandparent), so every walk ends, whatever other threads do meanwhile. */
__device__ __forceinline__ int find_root(int32_t* parent, int x) {
    while (true) {
        const int p = __atomic_load_n(&parent[x], __ATOMIC_RELAXED);
        if (p == x) return x;
        const int g = __atomic_load_n(&parent[p], __ATOMIC_RELAXED);
        if (g != p) __atomic_store_n(&parent[x], g, __ATOMIC_RELAXED); /* path halving */
        x = p;
    }
}

__device__ __forceinline__ void unite(int32_t* parent, int a, int b) {
    while (true) {
        a = find_root(parent, a);
        b = find_root(parent, b);
        if (a == b) return;
        const int hi = max(a, b), lo = min(a, b);
        if (atomicCAS(&parent[hi], hi, lo) == hi) return; /* hi was still a root: now it hangs below lo */
    }
}

__global__ __launch_bounds__(VMHIP_TILE) void vm_cluster_union_kernel(VmBatchDev B, VmDetectDev D) {
    const int tile = blockIdx.x;
    if (tile >= vm_row_tiles(B)) return; /* the grid may be sized for more tiles than the staged batch has */
    const int f = frame_of_row_tile(B.frames, B.n_frames, tile);
    const VmFrame& F = B.frames[f];
    const int V = F.n_cand > 0 ? B.frame_V[f] : 0; /* a frame without candidates has no rows */
    const int r = (tile - F.row_tile0) * VMHIP_TILE + (int) threadIdx.x;
    if (r >= V) return;
    const size_t base = (size_t) F.row_base;
    const int j = D.row_to_detection[base + r];
    if (j < 0) return;
    int32_t* parent = D.parent + base;
    const int32_t* nb = B.row_nb + (base + r) * B.nb_stride;
    for (int k = 0; k < F.nn; ++k) {
        const int n = nb[k];
        if (n >= V) continue; /* the null row: no visible neighbour there */
        const int jn = D.row_to_detection[base + n];
        if (jn >= 0 && jn != j) unite(parent, j, jn);
    }
}

__global__ __launch_bounds__(DETECT_THREADS) void vm_cluster_label_kernel(VmBatchDev B, VmDetectDev D) {
    __shared__ int scratch[DETECT_THREADS / 64];
    const int f = blockIdx.x;
    const size_t base = (size_t) B.frames[f].row_base;
    const int n = D.counts[2 * f];
    int32_t* parent = D.parent + base;
    int running = 0;
    /* roots, numbered in detection order; a root's number is parked in its cluster entry */
    for (int j0 = 0; j0 < n; j0 += DETECT_THREADS) {
        const int j = j0 + (int) threadIdx.x;
        const bool root = j < n && find_root(parent, j) == j;
        int total;
        const int id = running + block_rank(root, scratch, total);
        if (root) {
            D.cluster[base + j] = id;
            D.cluster_size[base + id] = 0;
            D.cluster_box[(base + id) * 4 + 0] = 0x7f800000; /* +inf as bits: pixels are not negative, so their */
            D.cluster_box[(base + id) * 4 + 1] = 0x7f800000; /* bit patterns order like the numbers            */
            D.cluster_box[(base + id) * 4 + 2] = 0;
            D.cluster_box[(base + id) * 4 + 3] = 0;
            D.cluster_sum[(base + id) * 2 + 0] = 0.0f;
            D.cluster_sum[(base + id) * 2 + 1] = 0.0f;
        }
        running += total;
    }
    __threadfence_block();
    __syncthreads();
    /* Label, and add every detection to its cluster's figures. A cluster can hold most of a frame, so the lanes of a
     * wave that belong to the same cluster combine their contribution first and one of them sends it: the atomics
     * on one cluster's words would otherwise queue up behind each other. */
    const int lane = threadIdx.x & 63;
    for (int j0 = 0; j0 < n; j0 += DETECT_THREADS) {
        const int j = j0 + (int) threadIdx.x;
        const bool active = j < n;
        int id = -1;
        float2 px = make_float2(0.0f, 0.0f);
        if (active) {
            const int root = find_root(parent, j);
            id = D.cluster[base + root]; /* a root's own entry never changes below */
            if (root != j) D.cluster[base + j] = id;
            px = D.pixel[base + j];
        }
        unsigned long long todo = __ballot(active);
        while (todo) {
            const int lead = __ffsll((long long) todo) - 1;
            const int lead_id = __shfl(id, lead);
            const bool mine = active && id == lead_id;
            const unsigned long long members = __ballot(mine);
            float lo_x = mine ? px.x : __uint_as_float(0x7f800000u), lo_y = mine ? px.y : __uint_as_float(0x7f800000u);
            float hi_x = mine ? px.x : 0.0f, hi_y = mine ? px.y : 0.0f;
            float sum_x = mine ? px.x : 0.0f, sum_y = mine ? px.y : 0.0f;
            for (int step = 1; step < 64; step <<= 1) {
                lo_x = fminf(lo_x, __shfl_xor(lo_x, step));
                lo_y = fminf(lo_y, __shfl_xor(lo_y, step));
                hi_x = fmaxf(hi_x, __shfl_xor(hi_x, step));
                hi_y = fmaxf(hi_y, __shfl_xor(hi_y, step));
                sum_x += __shfl_xor(sum_x, step);
                sum_y += __shfl_xor(sum_y, step);
            }
            if (lane == lead) {
                const size_t c = base + (size_t) lead_id;
                atomicAdd(&D.cluster_size[c], __popcll(members));
                atomicMin(&D.cluster_box[c * 4 + 0], (int32_t) __float_as_uint(lo_x));
                atomicMin(&D.cluster_box[c * 4 + 1], (int32_t) __float_as_uint(lo_y));
                atomicMax(&D.cluster_box[c * 4 + 2], (int32_t) __float_as_uint(hi_x));
                atomicMax(&D.cluster_box[c * 4 + 3], (int32_t) __float_as_uint(hi_y));
                atomicAdd(&D.cluster_sum[c * 2 + 0], sum_x);
                atomicAdd(&D.cluster_sum[c * 2 + 1], sum_y);
            }
            todo &= ~members;
        }
    }
    if (threadIdx.x == 0) D.counts[2 * f + 1] = running;
}

/* One block per frame copies the frame's detections and clusters into one dense block of 4-byte words, laid out as
 * node[ND] pixel[2 ND] probability[ND] cluster[ND] size[NC] box[4 NC] sum[2 NC] with the frames one after the other
 * inside every part, so that a single copy brings everything to the host. */
__global__ __launch_bounds__(DETECT_THREADS) void vm_detect_pack_kernel(VmBatchDev B, VmDetectDev D, uint32_t* packed, int total_d, int total_c) {
    const int f = blockIdx.x;
    int d0 = 0, c0 = 0;
    for (int g = 0; g < f; ++g) d0 += D.counts[2 * g], c0 += D.counts[2 * g + 1];
    const int nd = D.counts[2 * f], nc = D.counts[2 * f + 1];
    const size_t base = (size_t) B.frames[f].row_base;
    uint32_t* node = packed;
    uint32_t* pixel = node + total_d;
    uint32_t* probability = pixel + 2 * (size_t) total_d;
    uint32_t* cluster = probability + total_d;
    uint32_t* size = cluster + total_d;
    uint32_t* box = size + total_c;
    uint32_t* sum = box + 4 * (size_t) total_c;
    for (int j = (int) threadIdx.x; j < nd; j += DETECT_THREADS) {
        node[d0 + j] = (uint32_t) D.node[base + j];
        const float2 px = D.pixel[base + j];
        pixel[2 * (size_t) (d0 + j)] = __float_as_uint(px.x);
        pixel[2 * (size_t) (d0 + j) + 1] = __float_as_uint(px.y);
        probability[d0 + j] = __float_as_uint(D.probability[base + j]);
        cluster[d0 + j] = (uint32_t) D.cluster[base + j];
    }
    for (int c = (int) threadIdx.x; c < nc; c += DETECT_THREADS) {
        size[c0 + c] = (uint32_t) D.cluster_size[base + c];
        for (int k = 0; k < 4; ++k) box[4 * (size_t) (c0 + c) + k] = (uint32_t) D.cluster_box[(base + c) * 4 + k];
        for (int k = 0; k < 2; ++k) sum[2 * (size_t) (c0 + c) + k] = __float_as_uint(D.cluster_sum[(base + c) * 2 + k]);
    }
}

/* The results of all frames gathered into one block for a single download: segment g is `bytes` bytes at `src`, made of rows
 * of `row_bytes` that lie `src_stride` bytes apart (equal for a contiguous array), and goes to dst + dst_offset; the segments'
 * chunks of VM_PACK_CHUNK bytes are numbered through chunk_first. All sizes and offsets are multiples of 4, dst offsets of 256. */
__global__ __launch_bounds__(256) void vm_fetch_pack_kernel(const VmPackSegment* __restrict__ segments, int n_segments, uint8_t* __restrict__ dst) {
    int lo = 0, hi = n_segments - 1;
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (segments[mid].chunk_first <= (int) blockIdx.x) lo = mid;
        else hi = mid - 1;
    }
    const VmPackSegment g = segments[lo];
    const size_t begin = (size_t) ((int) blockIdx.x - g.chunk_first) * VM_PACK_CHUNK;
    const size_t end = begin + VM_PACK_CHUNK < g.bytes ? begin + VM_PACK_CHUNK : g.bytes;
    uint8_t* out = dst + g.dst_offset;
    if (g.row_bytes == g.src_stride && (reinterpret_cast<uintptr_t>(g.src) & 15) == 0) {
        const size_t vec_end = begin + ((end - begin) & ~(size_t) 15);
        for (size_t at = begin + (size_t) threadIdx.x * 16; at < vec_end; at += 256 * 16)
            *reinterpret_cast<uint4*>(out + at) = *reinterpret_cast<const uint4*>(g.src + at);
        for (size_t at = vec_end + (size_t) threadIdx.x * 4; at < end; at += 256 * 4)
            *reinterpret_cast<uint32_t*>(out + at) = *reinterpret_cast<const uint32_t*>(g.src + at);
    }
    else {
        for (size_t at = begin + (size_t) threadIdx.x * 4; at < end; at += 256 * 4) {
            const size_t row = at / g.row_bytes, in_row = at - row * g.row_bytes;
            *reinterpret_cast<uint32_t*>(out + at) = *reinterpret_cast<const uint32_t*>(g.src + row * g.src_stride + in_row);
        }
    }
}

}  // namespace

void vm_launch_fetch_pack(const VmPackSegment* segments, int n_segments, int n_chunks, void* dst, hipStream_t stream) {
    if (n_segments <= 0 || n_chunks <= 0) return;
    hipLaunchKernelGGL(vm_fetch_pack_kernel, dim3(n_chunks), dim3(256), 0, stream, segments, n_segments, static_cast<uint8_t*>(dst));
}

void vm_launch_detect_pack(const VmBatchDev& B, const VmDetectDev& D, uint32_t* packed, int total_d, int total_c, hipStream_t stream) {
    if (B.n_frames <= 0) return;
    hipLaunchKernelGGL(vm_detect_pack_kernel, dim3(B.n_frames), dim3(DETECT_THREADS), 0, stream, B, D, packed, total_d, total_c);
}

size_t vm_detect_workspace_bytes(size_t rows, int n_frames) { return rows * VM_DETECT_BYTES_PER_ROW + size_t(n_frames) * 8 + 256; }

void vm_detect_carve(void* workspace, size_t rows, int n_frames, VmDetectDev* D) {
    char* p = static_cast<char*>(workspace);
    auto take = [&](size_t bytes) {
        void* at = p;
        p += (bytes + 15) & ~size_t(15);
        return at;
    };
    D->cluster_box = static_cast<int32_t*>(take(rows * 16));
    D->pixel = static_cast<float2*>(take(rows * 8));
    D->cluster_sum = static_cast<float*>(take(rows * 8));
    D->node = static_cast<int32_t*>(take(rows * 4));
    D->probability = static_cast<float*>(take(rows * 4));
    D->cluster = static_cast<int32_t*>(take(rows * 4));
    D->row_to_detection = static_cast<int32_t*>(take(rows * 4));
    D->parent = static_cast<int32_t*>(take(rows * 4));
    D->cluster_size = static_cast<int32_t*>(take(rows * 4));
    D->counts = static_cast<int32_t*>(take(size_t(n_frames) * 8));
}

void vm_launch_detect(const VmBatchDev& B, const VmDetectDev& D, int clusters, hipStream_t stream) {
    if (B.n_frames <= 0) return;
    hipLaunchKernelGGL(vm_detect_kernel, dim3(B.n_frames), dim3(DETECT_THREADS), 0, stream, B, D);
    if (clusters) {
        if (B.n_row_tiles > 0) hipLaunchKernelGGL(vm_cluster_union_kernel, dim3(B.n_row_tiles), dim3(VMHIP_TILE), 0, stream, B, D);
        hipLaunchKernelGGL(vm_cluster_label_kernel, dim3(B.n_frames), dim3(DETECT_THREADS), 0, stream, B, D);
    }
}

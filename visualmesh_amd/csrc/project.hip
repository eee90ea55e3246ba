/*
 * project.hip - candidate projection, on-screen filter, order-preserving compaction, image sampling and
 * the local neighbourhood table, for gfx950 (wave64).
 *
 * This file is compiled with -ffp-contract=off: the lens projection and the bilinear weights must be
 * single IEEE binary32 operations in the reference's order, and acosf/sinf/tanf come from libm_exact.h,
 * which returns the host C library's bits. Pixel coordinates and sampled inputs are then bit-identical
 * to the CPU engine's. The ambiguity band below stays as a guard for hosts whose C library differs: a
 * node within 1/64 px of a screen edge is re-decided on the host, so the visible set cannot diverge.
 *
 * Kernels (one launch each per batch, grids over all frames of the batch):
 *   vm_project_kernel        candidate space: global index from the range table, pixel coordinate, keep
 *                            decision, per-wave keep mask (ballot), per-tile kept count, ambiguity list
 *   vm_compact_kernel        candidate space: exclusive prefix over tile counts + wave popcount prefix ->
 *                            ascending local row; writes pixel, global index, reverse lookup stamp and the
 *                            sampled 4-channel input row; the frame's last tile writes V and the null row
 *   vm_neighbourhood_kernel  row space: neighbour table through the stamped reverse lookup
 *   vm_publish_kernel        (after the network) counts and ambiguity lists into page-locked host memory; clears the
 *                            ambiguity counters and advances the run stamp for the next pass
 */
#include "vmhip_internal.h"

#include <type_traits>

#pragma clang fp contract(off)

#include "libm_exact.h"

namespace {

/* A pointer that was itself read from memory (a frame's tables, its image) is taken for one that might point into
 * LDS, and what it points to is then read through the slower generic path with a 64-bit vector address. These casts
 * say that it points to device memory. */
#define VM_GLOBAL __attribute__((address_space(1)))
template <typename T>
__device__ __forceinline__ const VM_GLOBAL T* in_device_memory(const T* p) {
    return (const VM_GLOBAL T*) p;
}
template <typename T>
__device__ __forceinline__ VM_GLOBAL T* in_device_memory(T* p) {
    return (VM_GLOBAL T*) p;
}
/* base[index] with the offset in Off's width */
template <typename T, typename Off>
__device__ __forceinline__ T read_element(const T* base, Off index) {
    return *reinterpret_cast<const VM_GLOBAL T*>((const VM_GLOBAL char*) reinterpret_cast<const char*>(base) + index * (Off) sizeof(T));
}
template <typename T, typename Off>
__device__ __forceinline__ void write_element(T* base, Off index, const T& value) {
    *reinterpret_cast<VM_GLOBAL T*>((VM_GLOBAL char*) reinterpret_cast<char*>(base) + index * (Off) sizeof(T)) = value;
}

__device__ __forceinline__ int find_frame_by_cand_tile(const VmFrame* frames, int n, int tile) {
    int lo = 0, hi = n - 1;
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (frames[mid].cand_tile0 <= tile) lo = mid;
        else hi = mid - 1;
    }
    return lo;
}
__device__ __forceinline__ int find_frame_by_row_tile(const VmFrame* frames, int n, int tile) {
    int lo = 0, hi = n - 1;
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (frames[mid].row_tile0 <= tile) lo = mid;
        else hi = mid - 1;
    }
    return lo;
}

/* candidate slot -> global node index: ranges are ascending, prefix[r] <= p < prefix[r+1] */
__device__ __forceinline__ int cand_to_global(const VmFrame& F, int p) {
    int lo = 0, hi = F.n_ranges - 1;
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (F.range_prefix[mid] <= p) lo = mid;
        else hi = mid - 1;
    }
    return F.range_first[lo] + (p - F.range_prefix[lo]);
}

/* The same for the 64 consecutive slots of a wave (p = the wave's first slot + lane): the range of the first slot is
 * taken from the batch's tile table or found once, by a search on wave-uniform values that the scalar unit carries out;
 * a lane then steps forward over the range boundaries that lie between that slot and its own - rarely more than one or two. */
__device__ __forceinline__ int cand_to_global_wave(const VmFrame& F, int p, int lane, int tile_range) {
    int lo = tile_range; /* the range of the tile's first slot, if the batch was staged with its tile tables */
    if (tile_range < 0) {
        const int p0 = __builtin_amdgcn_readfirstlane(p - lane);
        int hi = F.n_ranges - 1;
        lo = 0;
        while (lo < hi) {
            const int mid = (lo + hi + 1) >> 1;
            if (F.range_prefix[mid] <= p0) lo = mid;
            else hi = mid - 1;
        }
        lo = __builtin_amdgcn_readfirstlane(lo);
    }
    const VM_GLOBAL int32_t* const prefix = in_device_memory(F.range_prefix);
    const int n_ranges = F.n_ranges;
    int start = prefix[lo];
    while (lo + 1 < n_ranges) {
        const int next = prefix[lo + 1];
        if (next > p) break;
        start = next;
        ++lo;
    }
    return in_device_memory(F.range_first)[lo] + (p - start);
}

/* Lens projection, reference utility/projection.hpp:162-187 with utility/math.hpp's dot order. */
__device__ __forceinline__ float2 project_ray(const VmFrame& F, float rx, float ry, float rz) {
    const float c0 = F.Rco[2] * rz + (F.Rco[1] * ry + F.Rco[0] * rx);
    const float c1 = F.Rco[5] * rz + (F.Rco[4] * ry + F.Rco[3] * rx);
    const float c2 = F.Rco[8] * rz + (F.Rco[7] * ry + F.Rco[6] * rx);

    /* vm_acosf / vm_sinf / vm_tanf return the host C library's bits (libm_exact.h) */
    const float theta = vm_acosf(c0);
    const float rsin_theta = 1.0f / vm_sqrtf(1.0f - c0 * c0);
    float r_u;
    if (F.projection == VMHIP_RECTILINEAR) {
        r_u = F.focal * vm_tanf(fminf(fmaxf(theta, 0.0f), 1.57079637050628662109375f));
    }
    else if (F.projection == VMHIP_EQUISOLID) {
        r_u = 2.0f * F.focal * vm_sinf(theta * 0.5f);
    }
    else {
        r_u = F.focal * theta;
    }
    /* distortion polynomial: a double sum of float terms (the reference's literal 1.0). Without distortion every term
     * is a zero and the sum is exactly 1.0 unless a power of r_u overflowed (zero times infinity), so that a lens without
     * coefficients skips the double-precision steps and gets the same bits. */
    const float r2 = r_u * r_u;
    float r_d = r_u;
    const bool undistorted = F.ik[0] == 0.0f && F.ik[1] == 0.0f && F.ik[2] == 0.0f && F.ik[3] == 0.0f;
    if (!undistorted || !((r2 * r2) * (r2 * r2) < __builtin_inff())) {
        const double s = 1.0 + (double) (F.ik[0] * r2) + (double) (F.ik[1] * (r2 * r2)) + (double) (F.ik[2] * (r2 * r2) * r2)
                         + (double) (F.ik[3] * (r2 * r2) * (r2 * r2));
        r_d = (float) ((double) r_u * s);
    }

    float sx = 0.0f, sy = 0.0f;
    if (!(c0 >= 1.0f)) {
        sx = r_d * c1 * rsin_theta;
        sy = r_d * c2 * rsin_theta;
    }
    float2 px;
    px.x = ((float) F.width * 0.5f - sx) - F.centre_x;
    px.y = ((float) F.height * 0.5f - sy) - F.centre_y;
    return px;
}

__global__ void vm_libm_kernel(int which, const float* x, float* y, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const float v = x[i];
    y[i] = which == 0 ? vm_acosf(v) : which == 1 ? vm_sinf(v) : which == 2 ? vm_tanf(v) : vm_sqrtf(v);
}

/* plain streaming copy of 16-byte words: the yardstick the memory counters are scaled by */
__global__ __launch_bounds__(256) void vm_copy_probe_kernel(const float4* __restrict__ src, float4* __restrict__ dst, size_t n) {
    for (size_t i = (size_t) blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t) gridDim.x * blockDim.x) dst[i] = src[i];
}

/* A layer reduced to its memory traffic: every wave takes 64 rows at a time, reads their read_vec 16-byte pieces and
 * writes their write_vec 16-byte pieces (per 64 rows), both as whole cache lines, with nothing in between but an xor
 * that keeps the reads alive. What this reaches for a layer's mix of bytes read and written is what the memory system
 * gives a kernel of that shape at best. */
__global__ __launch_bounds__(256) void vm_stream_probe_kernel(const uint4* __restrict__ src, uint4* __restrict__ dst, size_t groups, int read_vec, int write_vec) {
    const int lane = threadIdx.x & 63;
    const size_t wave = ((size_t) blockIdx.x * blockDim.x + threadIdx.x) >> 6, n_waves = ((size_t) gridDim.x * blockDim.x) >> 6;
    for (size_t g = wave; g < groups; g += n_waves) {
        uint4 acc = make_uint4(0, 0, 0, 0);
        const uint4* in = src + g * (size_t) read_vec;
        for (int i = lane; i < read_vec; i += 64) {
            const uint4 v = in[i];
            acc.x ^= v.x, acc.y ^= v.y, acc.z ^= v.z, acc.w ^= v.w;
        }
        uint4* o = dst + g * (size_t) write_vec;
        for (int i = lane; i < write_vec; i += 64) o[i] = acc;
    }
}

/* Last kernel of a pass. What the host needs of the pass is written by the device straight into page-locked host memory
 * (block f: the head of frame f's ambiguity list; block 0 also the counts and the convolution kernel's count of waits that
 * ran out). A copy engine is not involved, so the few hundred bytes never queue behind another engine's 50 MB download.
 * Block 0 then prepares the next pass: the ambiguity counters (the second half of the counts) start from zero again,
 * and the run stamp advances, so that the stamps of this pass stop matching. (As a kernel of its own at the head of a pass
 * this cost 16 us: the pass's second kernel waited for the host to finish queueing it.) */
__global__ __launch_bounds__(64) void vm_publish_kernel(int32_t* __restrict__ counts, int n_counts, const int2* __restrict__ amb_list, int amb_stride,
                                                        int amb_head, const unsigned int* __restrict__ timeouts, uint32_t* __restrict__ epoch,
                                                        int32_t* host_counts, int2* host_amb, uint32_t* host_timeouts) {
    const int f = blockIdx.x;
    for (int t = threadIdx.x; t < amb_head; t += 64) host_amb[(size_t) f * amb_head + t] = amb_list[(size_t) f * amb_stride + t];
    if (f == 0) {
        for (int t = threadIdx.x; t < n_counts; t += 64) {
            host_counts[t] = counts[t];
            if (t >= n_counts / 2) counts[t] = 0;
        }
        if (threadIdx.x == 0) {
            *host_timeouts = timeouts ? *timeouts : 0u;
            *epoch += 1;
        }
    }
}

/* ---- lookup on the device: the host's walk of the cone tree (cpp/visualmesh/detail/cone_tree.hpp, itself after the
 * reference's mesh.hpp:499-595), one block per frame. Every test is the host's expression in the host's order, so
 * the set of covered nodes is the same; the host merges what it covers into maximal runs, which is what the scan over
 * the bit map at the end yields. ---- */
constexpr int LOOKUP_THREADS = 1024;

/* exclusive prefix of v over the block in thread order; total = the block's sum */
__device__ __forceinline__ int lookup_block_scan(int v, int* wave_total, int& total) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int scan = v;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const int up = __shfl_up(scan, d);
        if (lane >= d) scan += up;
    }
    __syncthreads(); /* wave_total may still be read from the call before */
    if (lane == 63) wave_total[wave] = scan;
    __syncthreads();
    int before = scan - v, sum = 0;
    for (int w = 0; w < LOOKUP_THREADS / 64; ++w) {
        if (w < wave) before += wave_total[w];
        sum += wave_total[w];
    }
    total = sum;
    return before;
}

/* a load that does not trust the CU's L1: the words read this way were written by other threads of the block, some
 * of them by atomics, which act on the L2 */
template <typename T>
__device__ __forceinline__ T lookup_read(const T* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

/* sets the bits [first, last): words that lie wholly inside belong to this range alone */
__device__ __forceinline__ void cover(uint32_t* covered, int first, int last) {
    if (last <= first) return;
    const int w0 = first >> 5, w1 = (last - 1) >> 5;
    const uint32_t head = 0xffffffffu << (first & 31), tail = 0xffffffffu >> (31 - ((last - 1) & 31));
    if (w0 == w1) {
        atomicOr(&covered[w0], head & tail);
        return;
    }
    atomicOr(&covered[w0], head);
    for (int w = w0 + 1; w < w1; ++w) covered[w] = 0xffffffffu;
    atomicOr(&covered[w1], tail);
}

__global__ __launch_bounds__(LOOKUP_THREADS) void vm_lookup_kernel(const VmLookupFrame* frames) {
    __shared__ int wave_total[LOOKUP_THREADS / 64];
    __shared__ int n_now, n_next, n_wide;
    __shared__ int2 wide[256]; /* ranges too long for one thread to cover by itself */
    const VmLookupFrame& L = frames[blockIdx.x];
    const VmFrame& F = L.frame;
    const int tid = threadIdx.x;
    const int words = (F.n_nodes + 31) >> 5;
    for (int i = tid; i < words; i += LOOKUP_THREADS) L.covered[i] = 0;
    if (tid == 0) {
        L.list[0][0] = 0;
        n_now = L.n_elements > 0 ? 1 : 0;
        n_next = 0;
        n_wide = 0;
    }
    __syncthreads();

    const float ox = F.Rco[0], oy = F.Rco[1], oz = F.Rco[2]; /* the optical axis in observation-plane space */
    const float W = (float) F.width, H = (float) F.height;
    auto on_screen = [&](const float2 px) { return 0.0f <= px.x && px.x + 1.0f <= W && 0.0f <= px.y && px.y + 1.0f <= H; };
    int cur = 0;
    while (n_now > 0) {
        const int n = n_now;
        for (int i = tid; i < n; i += LOOKUP_THREADS) {
            const VmTreeElement e = L.tree[lookup_read(&L.list[cur][i])];
            /* field-of-view cone first: cos(a -/+ b) by the compound angle formula */
            const float along = oz * e.axis[2] + (oy * e.axis[1] + ox * e.axis[0]);
            bool outside = along < L.cos_half_fov * e.c - L.sin_half_fov * e.s;
            bool inside = along > L.cos_half_fov * e.c + L.sin_half_fov * e.s;
            if (!outside && inside) {
                const bool axis_on_screen = on_screen(project_ray(F, e.axis[0], e.axis[1], e.axis[2]));
                float edge_along[4];
                bool beyond = false;
                for (int k = 0; k < 4; ++k) {
                    edge_along[k] = e.axis[2] * L.edge[k][2] + (e.axis[1] * L.edge[k][1] + e.axis[0] * L.edge[k][0]);
                    beyond = beyond || edge_along[k] > L.edge[k][3] * e.c + L.edge[k][4] * e.s;
                }
                if (!axis_on_screen && beyond) {
                    inside = false;
                    outside = true;
                }
                else {
                    bool clear = true;
                    for (int k = 0; k < 4; ++k) clear = clear && edge_along[k] < L.edge[k][3] * e.c - L.edge[k][4] * e.s;
                    inside = axis_on_screen && clear;
                    outside = false;
                }
            }
            if (inside) {
                if (e.last - e.first > 2048) {
                    const int at = atomicAdd(&n_wide, 1);
                    if (at < 256) wide[at] = make_int2(e.first, e.last);
                    else cover(L.covered, e.first, e.last);
                }
                else {
                    cover(L.covered, e.first, e.last);
                }
            }
            else if (outside) {
            }
            else if (e.child[0] < 0) {
                for (int g = e.first; g < e.last; ++g) {
                    const float* r = F.rays + (size_t) g * 3;
                    const bool seen = oz * r[2] + (oy * r[1] + ox * r[0]) > L.cos_half_fov && on_screen(project_ray(F, r[0], r[1], r[2]));
                    if (seen) atomicOr(&L.covered[g >> 5], 1u << (g & 31));
                }
            }
            else {
                const int at = atomicAdd(&n_next, 2);
                L.list[cur ^ 1][at] = e.child[0];
                L.list[cur ^ 1][at + 1] = e.child[1];
            }
        }
        __syncthreads();
        if (tid == 0) {
            n_now = n_next;
            n_next = 0;
        }
        cur ^= 1;
        __syncthreads();
    }
    /* the long ranges, by everybody (whole words only; their ends as above) */
    const int n_long = min(n_wide, 256);
    for (int k = 0; k < n_long; ++k) {
        const int first = wide[k].x, last = wide[k].y;
        const int w0 = (first + 31) >> 5, w1 = last >> 5; /* whole words [w0, w1) */
        for (int w = w0 + tid; w < w1; w += LOOKUP_THREADS) L.covered[w] = 0xffffffffu;
        if (tid == 0) { /* such a range spans many words, so w0 < w1 */
            cover(L.covered, first, w0 << 5);
            cover(L.covered, w1 << 5, last);
        }
    }
    __syncthreads();

    /* maximal runs of covered nodes, in order: their starts into list[0], their ends into list[1] */
    int runs = 0, run_ends = 0;
    for (int base = 0; base < words; base += LOOKUP_THREADS) {
        const int w = base + tid;
        uint32_t v = 0, starts = 0, ends = 0;
        if (w < words) {
            v = lookup_read(&L.covered[w]);
            const uint32_t below = w > 0 ? lookup_read(&L.covered[w - 1]) >> 31 : 0u;
            const uint32_t above = w + 1 < words ? lookup_read(&L.covered[w + 1]) & 1u : 0u;
            starts = v & ~((v << 1) | below);
            ends = v & ~((v >> 1) | (above << 31));
        }
        int total_starts, total_ends;
        int at = runs + lookup_block_scan(__popc(starts), wave_total, total_starts);
        int at_end = run_ends + lookup_block_scan(__popc(ends), wave_total, total_ends);
        while (starts) {
            const int bit = __ffs((int) starts) - 1;
            if (at < L.capacity) L.list[0][at] = (w << 5) + bit;
            ++at;
            starts &= starts - 1;
        }
        while (ends) {
            const int bit = __ffs((int) ends) - 1;
            if (at_end < L.capacity) L.list[1][at_end] = (w << 5) + bit + 1;
            ++at_end;
            ends &= ends - 1;
        }
        runs += total_starts;
        run_ends += total_ends;
    }
    __syncthreads();
    __shared__ int dense_at;
    if (runs > L.capacity) { /* cannot happen with capacity = n_elements, but nothing is written past it either */
        if (tid == 0) L.verdict[0] = -1, L.verdict[1] = 0, L.verdict[2] = 0;
        return;
    }
    if (tid == 0) dense_at = atomicAdd(L.cursor, 2 * runs + 1);
    __syncthreads();
    int32_t* const first_out = L.dense + dense_at;
    int32_t* const prefix_out = first_out + runs;
    int candidates = 0;
    for (int base = 0; base < runs; base += LOOKUP_THREADS) {
        const int k = base + tid;
        int length = 0, first = 0;
        if (k < runs) {
            first = lookup_read(&L.list[0][k]);
            length = lookup_read(&L.list[1][k]) - first;
        }
        int total;
        const int before = candidates + lookup_block_scan(length, wave_total, total);
        if (k < runs) {
            first_out[k] = first;
            prefix_out[k] = before;
        }
        candidates += total;
    }
    if (tid == 0) {
        prefix_out[runs] = candidates;
        L.verdict[0] = runs;
        L.verdict[1] = candidates;
        L.verdict[2] = dense_at;
    }
}

/* ---- the lookup as a training pipeline wants it (reference tensorflow/lookup.cpp:186-249): for every node of the
 * frame's ranges its unit vector and a row [own position, positions of its neighbours], positions counted along the
 * ranges; a neighbour outside the ranges is the most negative int32 (HARD edges) or the node itself (SAME edges,
 * training/dataset/projection/visual_mesh.py:82-89). Pixel coordinates go along, as project() gives them. ---- */
__global__ __launch_bounds__(VMHIP_TILE) void vm_lookup_export_kernel(VmBatchDev B, int same_edges, float* __restrict__ vectors,
                                                                       int32_t* __restrict__ graph, float2* __restrict__ pixels) {
    const int tile = blockIdx.x;
    if (tile >= vm_cand_tiles(B)) return; /* the grid may be sized for more tiles than the staged batch has */
    const int f = find_frame_by_cand_tile(B.frames, B.n_frames, tile);
    const VmFrame& F = B.frames[f];
    const int p = (tile - F.cand_tile0) * VMHIP_TILE + threadIdx.x;
    if (p >= F.n_cand) return;
    const int g = cand_to_global(F, p);
    const size_t slot = (size_t) F.cand_base + p;
    const float* r = F.rays + (size_t) g * 3;
    vectors[slot * 3 + 0] = r[0];
    vectors[slot * 3 + 1] = r[1];
    vectors[slot * 3 + 2] = r[2];
    pixels[slot] = project_ray(F, r[0], r[1], r[2]);
    int32_t* row = graph + (size_t) F.cand_base * (B.nb_stride + 1) + (size_t) p * (F.nn + 1);
    row[0] = p;
    for (int j = 0; j < F.nn; ++j) {
        const int n = F.nbr[(size_t) g * F.nn + j];
        /* the last range that starts at or before n, if any, and whether n lies inside it */
        int lo = 0, hi = F.n_ranges - 1;
        while (lo < hi) {
            const int mid = (lo + hi + 1) >> 1;
            if (F.range_first[mid] <= n) lo = mid;
            else hi = mid - 1;
        }
        const int first = F.range_first[lo], length = F.range_prefix[lo + 1] - F.range_prefix[lo];
        const bool found = n >= first && n - first < length;
        row[j + 1] = found ? F.range_prefix[lo] + (n - first) : same_edges ? p : (int32_t) 0x80000000;
    }
}

__global__ __launch_bounds__(VMHIP_TILE) void vm_project_kernel(VmBatchDev B) {
    __shared__ int wave_count[VMHIP_TILE / 64];
    const int tile = blockIdx.x;
    if (tile >= vm_cand_tiles(B)) return; /* the grid may be sized for more tiles than the staged batch has */
    int f, tile_range = -1;
    if (B.cand_tile_info) {
        const int2 info = B.cand_tile_info[tile];
        f = info.x, tile_range = info.y;
    }
    else {
        f = find_frame_by_cand_tile(B.frames, B.n_frames, tile);
    }
    const VmFrame& F = B.frames[f];
    /* the frame's placement as values: read through F again after a store, it would be fetched again */
    const int cand_base = F.cand_base, cand_tile0 = F.cand_tile0;
    const int p = (tile - cand_tile0) * VMHIP_TILE + threadIdx.x;
    const bool valid = p < F.n_cand;

    bool keep = false;
    float2 px = make_float2(0.0f, 0.0f);
    if (valid) {
        /* the host's overruling decisions for this wave's candidates: read ahead of the arithmetic they do not depend on */
        const size_t word = (size_t) (cand_base + p) >> 6;
        const uint64_t force_valid = in_device_memory(F.force_valid)[word];
        const int g = cand_to_global_wave(F, p, threadIdx.x & 63, tile_range);
        const VM_GLOBAL float* r = in_device_memory(F.rays) + (size_t) g * 3;
        px = project_ray(F, r[0], r[1], r[2]);
        px.x += B.px_error, px.y += B.px_error; /* zero outside tests of the edge guard */
        const float W = (float) F.width, H = (float) F.height;
        /* strict test of the CPU engine, engine/cpu/engine.hpp:116-117 */
        keep = 0.0f <= px.x && px.x + 1.0f < W && 0.0f <= px.y && px.y + 1.0f < H;

        /* distance to the nearest decision boundary; NaN counts as ambiguous */
        const float d = fminf(fminf(fabsf(px.x), fabsf(px.x + 1.0f - W)), fminf(fabsf(px.y), fabsf(px.y + 1.0f - H)));
        const bool ambiguous = !(d >= B.amb_eps);

        const uint64_t bit = 1ull << (threadIdx.x & 63);
        const bool forced = (force_valid & bit) != 0;
        if (forced) { keep = (in_device_memory(F.force_keep)[word] & bit) != 0; }
        else if (ambiguous) {
            const int slot = atomicAdd(&B.amb_count[f], 1);
            if (slot < VMHIP_AMB_CAP) B.amb_list[(size_t) f * VMHIP_AMB_CAP + slot] = make_int2(p, keep ? 1 : 0);
        }
        B.cand_px[(size_t) cand_base + p] = px;
        B.cand_g[(size_t) cand_base + p] = g;
    }

    const uint64_t mask = __ballot(keep);
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) {
        B.cand_keep[((size_t) cand_base >> 6) + (size_t) (tile - cand_tile0) * (VMHIP_TILE / 64) + wave] = mask;
        wave_count[wave] = __popcll(mask);
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        int total = 0;
        for (int w = 0; w < VMHIP_TILE / 64; ++w) total += wave_count[w];
        B.tile_count[tile] = total;
    }
}

/* ---- image sampling: reference engine/cpu/pixel.hpp and bayer.hpp ---- */
#define INV255 0.0039215688593685626983642578125f /* float(1.0 / 255.0) */

__device__ __forceinline__ float4 texel_packed(const VmFrame& F, int x, int y) {
    const size_t idx = (size_t) y * F.width + x;
    float4 o;
    switch (F.fmt) {
        case VMHIP_FMT_RGBA: {
            const uint32_t v = in_device_memory(reinterpret_cast<const uint32_t*>(F.image))[idx];
            o = make_float4((float) (v & 0xff) * INV255, (float) ((v >> 8) & 0xff) * INV255,
                            (float) ((v >> 16) & 0xff) * INV255, (float) (v >> 24) * INV255);
        } break;
        case VMHIP_FMT_BGRA: {
            const uint32_t v = in_device_memory(reinterpret_cast<const uint32_t*>(F.image))[idx];
            o = make_float4((float) ((v >> 16) & 0xff) * INV255, (float) ((v >> 8) & 0xff) * INV255,
                            (float) (v & 0xff) * INV255, (float) (v >> 24) * INV255);
        } break;
        case VMHIP_FMT_RGB3: {
            const VM_GLOBAL uint8_t* b = in_device_memory(F.image) + idx * 3;
            o = make_float4((float) b[0] * INV255, (float) b[1] * INV255, (float) b[2] * INV255, 1.0f);
        } break;
        case VMHIP_FMT_BGR3: {
            const VM_GLOBAL uint8_t* b = in_device_memory(F.image) + idx * 3;
            o = make_float4((float) b[2] * INV255, (float) b[1] * INV255, (float) b[0] * INV255, 1.0f);
        } break;
        default: { /* GRAY */
            const float v = (float) in_device_memory(F.image)[idx] * INV255;
            o = make_float4(v, v, v, 1.0f);
        } break;
    }
    return o;
}

/* Malvar-He-Cutler demosaic of the 5x5 patch whose top-left corner is (ox, oy) inside the 6x6 union u.
 * Integer arithmetic with truncating division by 64 and no clamp (bayer.hpp:95-108). type: 0 R, 1 GR, 2 GB, 3 B */
template <int OX, int OY>
__device__ __forceinline__ float4 demosaic_at(const int (&u)[6][6], int type) {
#define P(r, c) u[OY + (r)][OX + (c)]
    const int centre = P(2, 2);
    int red, green, blue;
    if (type == 0 || type == 3) {
        const int arms = P(0, 2) + P(2, 0) + P(2, 4) + P(4, 2);
        const int cross = (-8 * arms + 16 * (P(1, 2) + P(2, 1) + P(2, 3) + P(3, 2)) + 32 * centre) / 64;
        const int checker = (-12 * arms + 16 * (P(1, 1) + P(1, 3) + P(3, 1) + P(3, 3)) + 48 * centre) / 64;
        green = cross;
        red = type == 0 ? centre : checker;
        blue = type == 0 ? checker : centre;
    }
    else {
        const int diag = P(1, 1) + P(1, 3) + P(3, 1) + P(3, 3);
        const int horiz = (4 * (P(0, 2) + P(4, 2)) - 8 * diag - 8 * (P(2, 0) + P(2, 4)) + 32 * (P(2, 1) + P(2, 3)) + 40 * centre) / 64;
        const int vert = (-8 * (P(0, 2) + P(4, 2)) - 8 * diag + 32 * (P(1, 2) + P(3, 2)) + 4 * (P(2, 0) + P(2, 4)) + 40 * centre) / 64;
        green = centre;
        red = type == 1 ? horiz : vert;
        blue = type == 1 ? vert : horiz;
    }
#undef P
    return make_float4((float) red * INV255, (float) green * INV255, (float) blue * INV255, (float) 255 * INV255);
}

__device__ __forceinline__ int bayer_type(int fmt, int x, int y) {
    /* pattern letters in (row, col) order: index = row*2 + col; 0 R, 1 GR, 2 GB, 3 B (bayer.hpp:140-155) */
    const int i = ((y & 1) << 1) | (x & 1);
    switch (fmt) {
        case VMHIP_FMT_GRBG: return (0x2301 >> (i * 4)) & 0xf; /* GR R B GB */
        case VMHIP_FMT_RGGB: return (0x3210 >> (i * 4)) & 0xf; /* R GR GB B */
        case VMHIP_FMT_GBRG: return (0x1032 >> (i * 4)) & 0xf; /* GB B R GR */
        default: return (0x0123 >> (i * 4)) & 0xf;             /* BGGR: B GB GR R */
    }
}

/* bilinear interpolation of the four surrounding texels, reference engine/cpu/pixel.hpp:115-144. The
 * on-screen filter guarantees 0 <= x and x + 1 < width, so x2 = x1 + 1 and the reference's division by
 * (x2 - x1) is a division by one. */
__device__ __forceinline__ float4 sample_image(const VmFrame& F, float2 px) {
    const int x1 = max((int) floorf(px.x), 0);
    const int y1 = max((int) floorf(px.y), 0);
    const int x2 = min(x1 + 1, F.width - 1);
    const int y2 = min(y1 + 1, F.height - 1);
    float4 q1, q2, q3, q4;
    if (F.fmt >= VMHIP_FMT_GRBG && F.fmt <= VMHIP_FMT_BGGR) {
        int u[6][6];
#pragma unroll
        for (int r = 0; r < 6; ++r) {
            const int yc = min(max(y1 - 2 + r, 0), F.height - 1);
#pragma unroll
            for (int c = 0; c < 6; ++c) {
                const int xc = min(max(x1 - 2 + c, 0), F.width - 1);
                u[r][c] = in_device_memory(F.image)[(size_t) yc * F.width + xc];
            }
        }
        /* x2 == x1 or y2 == y1 only on the last column/row, which the filter excludes; handle anyway */
        q1 = demosaic_at<0, 0>(u, bayer_type(F.fmt, x1, y1));
        q2 = x2 > x1 ? demosaic_at<1, 0>(u, bayer_type(F.fmt, x2, y1)) : q1;
        q3 = y2 > y1 ? demosaic_at<0, 1>(u, bayer_type(F.fmt, x1, y2)) : q1;
        q4 = (x2 > x1 && y2 > y1) ? demosaic_at<1, 1>(u, bayer_type(F.fmt, x2, y2)) : (x2 > x1 ? q2 : q3);
    }
    else {
        q1 = texel_packed(F, x1, y1);
        q2 = texel_packed(F, x2, y1);
        q3 = texel_packed(F, x1, y2);
        q4 = texel_packed(F, x2, y2);
    }
    const float wxa = ((float) x2 - px.x) / (float) (x2 - x1), wxb = (px.x - (float) x1) / (float) (x2 - x1);
    const float wya = ((float) y2 - px.y) / (float) (y2 - y1), wyb = (px.y - (float) y1) / (float) (y2 - y1);
    float4 o;
    {
        const float r1 = q1.x * wxa + q2.x * wxb, r2 = q3.x * wxa + q4.x * wxb;
        o.x = r1 * wya + r2 * wyb;
    }
    {
        const float r1 = q1.y * wxa + q2.y * wxb, r2 = q3.y * wxa + q4.y * wxb;
        o.y = r1 * wya + r2 * wyb;
    }
    {
        const float r1 = q1.z * wxa + q2.z * wxb, r2 = q3.z * wxa + q4.z * wxb;
        o.z = r1 * wya + r2 * wyb;
    }
    {
        const float r1 = q1.w * wxa + q2.w * wxb, r2 = q3.w * wxa + q4.w * wxb;
        o.w = r1 * wya + r2 * wyb;
    }
    return o;
}

__global__ __launch_bounds__(VMHIP_TILE) void vm_compact_kernel(VmBatchDev B, float4* feat, int classify) {
    __shared__ int partial[VMHIP_TILE / 64];
    __shared__ int wave_count[VMHIP_TILE / 64];
    const int tile = blockIdx.x;
    if (tile >= vm_cand_tiles(B)) return;
    const int f = B.cand_tile_info ? B.cand_tile_info[tile].x : find_frame_by_cand_tile(B.frames, B.n_frames, tile);
    const VmFrame& F = B.frames[f];
    /* the frame's placement as values: read through F again after a store, it would be fetched again */
    const int cand_base = F.cand_base, cand_tile0 = F.cand_tile0, cand_tiles = F.cand_tiles, row_base = F.row_base;
    const int t_local = tile - cand_tile0;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;

    /* What a kept candidate brings along does not depend on where it lands: its node, its pixel and the image sample are
     * read and worked out first, so that these reads are under way while the block counts the kept candidates before it. */
    const uint64_t mask = B.cand_keep[((size_t) cand_base >> 6) + (size_t) t_local * (VMHIP_TILE / 64) + wave];
    const bool kept = (mask >> lane) & 1ull;
    const int p = t_local * VMHIP_TILE + threadIdx.x;
    int g = 0;
    float2 px = make_float2(0.0f, 0.0f);
    float4 sample = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    if (kept) {
        g = B.cand_g[(size_t) cand_base + p];
        px = B.cand_px[(size_t) cand_base + p];
        if (classify) sample = sample_image(F, px);
    }

    /* kept candidates in this frame's earlier tiles */
    int sum = 0;
    for (int i = threadIdx.x; i < t_local; i += VMHIP_TILE) sum += B.tile_count[cand_tile0 + i];
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) sum += __shfl_xor(sum, o);
    if (lane == 0) {
        partial[wave] = sum;
        wave_count[wave] = __popcll(mask);
    }
    __syncthreads();
    int base = 0, before = 0, total = 0;
#pragma unroll
    for (int w = 0; w < VMHIP_TILE / 64; ++w) {
        base += partial[w];
        if (w < wave) before += wave_count[w];
        total += wave_count[w];
    }

    if (kept) {
        const int local = base + before + __popcll(mask & ((1ull << lane) - 1ull));
        const size_t row = (size_t) row_base + local;
        B.row_px[row] = px;
        B.row_gidx[row] = g;
        in_device_memory(F.r_lookup)[g] = (*B.epoch << B.stamp_row_bits) | (uint32_t) local;
        if (classify) feat[row] = sample;
    }
    if (t_local == cand_tiles - 1 && threadIdx.x == 0) {
        const int V = base + total;
        B.frame_V[f] = V;
        /* the off-screen row, engine/cpu/engine.hpp:205-206 */
        if (classify) feat[(size_t) row_base + V] = make_float4(-1.0f, -1.0f, -1.0f, -1.0f);
    }
}

/* reference engine/cpu/engine.hpp:127-143: one thread per (row, neighbour).
 *
 * When the batch carries tile-local tables the block also builds them for its tile: the neighbours that live in
 * other tiles are deduplicated through an open-addressing hash in LDS, the thread that enters a row first takes the
 * next halo slot from a counter, and every neighbour is rewritten as a position in "own tile rows, then halo
 * slots". Which row gets which halo slot depends on the order the atomics land in and differs from run to run;
 * the rows that a slot stands for, and so every result computed through the tables, do not.
 *
 * WIDE = false addresses the frame's tables with 32-bit byte offsets from wave-uniform bases (an address is then a
 * scalar register pair plus one vector register, and the 64-bit vector arithmetic that was a third of this kernel's
 * instructions is gone); the host picks WIDE = true for a batch with a table of 4 GiB or more.
 *
 * CB > 0: the block also computes the network's first layer for its tile (reference engine/cpu/engine.hpp:213-264 for the
 * group's first dense layer: gather of [self, neighbours] over the 4-channel sampled rows, dense, bias, activation),
 * CB column blocks of 16 output channels. At this point the tile's neighbour rows are in registers and the rows it
 * gathers are 16 bytes each: the layer's 28 (36) input values per row are requested as soon as the neighbours are known
 * and arrive while the block builds its tile-local tables, so the layer costs neither a launch of its own nor a second
 * read of the neighbour table. v_mfma_f32_16x16x4_f32: A = weights (lane l: W[4 slot + l / 16][16 cb + l % 16], the order
 * vm_mfma_permute_weights stores), B = one gathered row per step (lane l: channel l / 16 of the row's source), D: lane l
 * holds channels 16 cb + 4 (l / 16) + {0..3} of row l % 16, one 16-byte store. */
#define NB_HASH 2048 /* >= the most out-of-tile neighbours a tile can have (256 rows x 8) */
typedef float nbc_v4f __attribute__((ext_vector_type(4)));
typedef uint32_t nbc_v4u __attribute__((ext_vector_type(4)));
typedef int nbc_v2i __attribute__((ext_vector_type(2)));
/* selu as the convolution kernels compute it: hardware exponential on the negative branch (<= 3e-7 absolute error) */
__device__ __forceinline__ float nbc_selu(float s) {
    const float lambda = 1.0507009873554804934193349852946f;
    const float alpha = 1.6732632423543772848170429916717f;
    return lambda * (s >= 0.0f ? s : __builtin_fmaf(alpha, __builtin_amdgcn_exp2f(s * 1.44269504088896340736f), -alpha));
}
template <bool WIDE, int NN, int CB>
__global__ __launch_bounds__(VMHIP_TILE, CB == 1 ? (NN <= 6 ? 8 : 6) : CB == 2 ? 5 : 1) void vm_neighbourhood_kernel(VmBatchDev B, VmLayerDev L, const float* __restrict__ feat, float* __restrict__ layer_out) {
    static_assert(CB == 0 || (NN > 0 && NN <= VMHIP_NBL_STRIDE), "the fused first layer knows its neighbour count");
    using Off = typename std::conditional<WIDE, size_t, uint32_t>::type;
    __shared__ __align__(16) uint32_t h_key[NB_HASH];
    __shared__ int halo_count; /* halo slots handed out so far */
    __shared__ uint16_t h_dense[NB_HASH];
    __shared__ __align__(16) uint16_t nbl_rows[VMHIP_TILE][VMHIP_NBL_STRIDE]; /* the tile's positions, stored row by row at the end */
    /* CB > 0: the frame-local row of every halo slot. The sampled rows the layer gathers (the tile's 256, then its halo
     * rows, 16 bytes each) are staged where the hash table lay, once nothing reads it any more. */
    __shared__ uint32_t halo_list[CB > 0 ? VMHIP_HALO_MAX : 1];
    static_assert(sizeof(h_key) >= (VMHIP_TILE + VMHIP_HALO_MAX) * 16, "the staged rows fit the hash table's memory");

    const int tile = blockIdx.x;
    if (tile >= vm_row_tiles(B)) return;
    const int f = B.row_tile_frame ? B.row_tile_frame[tile] : find_frame_by_row_tile(B.frames, B.n_frames, tile);
    const VmFrame& F = B.frames[f];
    const int V = B.frame_V[f];
    /* the frame's fields as values: read through F again after a store, they would be fetched again */
    const int nn = NN > 0 ? NN : F.nn, n_nodes = F.n_nodes, row_base = F.row_base;
    const int row0 = (tile - F.row_tile0) * VMHIP_TILE;
    const bool tables = B.row_nbl != nullptr;
    const uint32_t epoch = *B.epoch, row_mask = (1u << B.stamp_row_bits) - 1u;
    const int n_rows = max(0, min(VMHIP_TILE, V + 1 - row0));
    if (n_rows == 0) {
        if (tables && threadIdx.x == 0) B.tile_desc[tile] = make_int4(row_base + row0, 0, 0, row_base);
        return;
    }
    constexpr uint32_t EMPTY = 0xffffffffu;
    auto hash = [](uint32_t key) { return (key * 2654435761u) >> 21; }; /* 11 bits */
    if (tables) {
        for (int e = threadIdx.x * 4; e < NB_HASH; e += VMHIP_TILE * 4) *reinterpret_cast<uint4*>(&h_key[e]) = make_uint4(EMPTY, EMPTY, EMPTY, EMPTY);
        if (threadIdx.x == 0) halo_count = 0;
        __syncthreads();
    }

    /* the frame's parts of the tables, wave-uniform */
    const int32_t* const gidx = B.row_gidx + row_base;
    int32_t* const nb_out = B.row_nb + (size_t) row_base * B.nb_stride;
    const int32_t* const nbr = F.nbr;
    const uint32_t* const lookup = F.r_lookup;
    const Off nb_stride = (Off) B.nb_stride;

    /* (row, neighbour) items are dealt round-robin to the threads, VMHIP_TILE at a time, so that a thread has at most nn
     * of them; it takes them MAX_ITEMS at a time and keeps their results in registers between the passes (the tables
     * are only built for nn <= VMHIP_NBL_STRIDE, one round). NN > 0: every frame of the batch has NN neighbours per node, and
     * the rounds have no idle items; NN = 0: whatever the frame has, eight at a time, with the
     * item -> row division by nn as a multiplication by ceil(2^32 / nn), exact while item * nn < 2^32. */
    const int n_items = n_rows * nn;
    const uint32_t nn_magic = nn > 1 ? 0xffffffffu / (uint32_t) nn + 1u : 0u;
    auto row_of = [&](int it) { return NN > 0 ? it / (NN > 0 ? NN : 1) : nn > 1 ? (int) __umulhi((uint32_t) it, nn_magic) : it; };
    constexpr int MAX_ITEMS = NN > 0 ? NN : VMHIP_NBL_STRIDE;
    int outs[MAX_ITEMS];

    /* Items k0 .. k0 + MAX_ITEMS - 1 of this thread. The three dependent reads of an item (row -> node, node -> neighbour
     * node, neighbour node -> its row) go level by level over all the items, so that the items' reads are in flight together
     * and no store or branch stands between them: an item that does not exist, or that belongs to the null row, reads what
     * the frame's last row reads, and its result is not used. */
    auto resolve = [&](int k0) {
        bool live[MAX_ITEMS];
        uint32_t stamp[MAX_ITEMS];
        int item_row[MAX_ITEMS], item_slot[MAX_ITEMS];
#pragma unroll
        for (int k = 0; k < MAX_ITEMS; ++k) {
            const int it = threadIdx.x + (k0 + k) * VMHIP_TILE;
            const int r = row_of(it);
            item_row[k] = row0 + r;
            item_slot[k] = it - r * nn;
            live[k] = it < n_items;
            stamp[k] = 0u; /* zero carries no run's stamp: runs count from one */
        }
        if (V > 0) {
            int node[MAX_ITEMS];
#pragma unroll
            for (int k = 0; k < MAX_ITEMS; ++k) node[k] = read_element(gidx, (Off) min(item_row[k], V - 1));
#pragma unroll
            for (int k = 0; k < MAX_ITEMS; ++k) node[k] = min(read_element(nbr, (Off) node[k] * (Off) nn + (Off) item_slot[k]), n_nodes);
#pragma unroll
            for (int k = 0; k < MAX_ITEMS; ++k) stamp[k] = read_element(lookup, (Off) node[k]);
        }
#pragma unroll
        for (int k = 0; k < MAX_ITEMS; ++k) {
            outs[k] = -1;
            if (live[k]) {
                const bool found = item_row[k] < V && (stamp[k] >> B.stamp_row_bits) == epoch;
                const int out = found ? (int) (stamp[k] & row_mask) : V;
                write_element(nb_out, (Off) item_row[k] * nb_stride + (Off) item_slot[k], out);
                outs[k] = out;
            }
        }
    };
    if (!tables) {
        for (int k0 = 0; k0 < nn; k0 += MAX_ITEMS) resolve(k0);
        return;
    }
    /* With the tables, and the neighbour count known at compile time, a thread takes one row and all its neighbours
     * (PER_ROW): the row's node is read once, its neighbours are NN consecutive words of the mesh's table (read and
     * written two at a time), no item needs a division to find its row, and the row's eight table entries are packed in
     * registers and stored with one instruction. A wave's reads and writes of the two tables are contiguous either way.
     * Threads past the tile's rows redo its last row and store nothing. */
    constexpr bool PER_ROW = NN > 0 && NN % 2 == 0;
    const bool have_row = (int) threadIdx.x < n_rows;
    if constexpr (PER_ROW) {
        const int row = row0 + min((int) threadIdx.x, n_rows - 1);
        uint32_t stamp[NN];
#pragma unroll
        for (int k = 0; k < NN; ++k) stamp[k] = 0u; /* zero carries no run's stamp: runs count from one */
        if (V > 0) {
            const int node = read_element(gidx, (Off) min(row, V - 1));
            int nb[NN];
#pragma unroll
            for (int j = 0; j < NN / 2; ++j) {
                const nbc_v2i two = read_element(reinterpret_cast<const nbc_v2i*>(nbr), (Off) node * (Off) (NN / 2) + (Off) j);
                nb[2 * j] = min(two.x, n_nodes), nb[2 * j + 1] = min(two.y, n_nodes);
            }
#pragma unroll
            for (int k = 0; k < NN; ++k) stamp[k] = read_element(lookup, (Off) nb[k]);
        }
#pragma unroll
        for (int k = 0; k < NN; ++k) {
            const bool found = row < V && (stamp[k] >> B.stamp_row_bits) == epoch;
            outs[k] = have_row ? (found ? (int) (stamp[k] & row_mask) : V) : -1;
        }
        if (have_row) {
            if (B.nb_stride == NN) {
#pragma unroll
                for (int j = 0; j < NN / 2; ++j) write_element(reinterpret_cast<nbc_v2i*>(nb_out), (Off) row * (Off) (NN / 2) + (Off) j, nbc_v2i{outs[2 * j], outs[2 * j + 1]});
            }
            else {
#pragma unroll
                for (int k = 0; k < NN; ++k) write_element(nb_out, (Off) row * nb_stride + (Off) k, outs[k]);
            }
        }
    }
    else {
        resolve(0);
    }

    /* ---- first layer, part one: request what the contraction will read ---- */
    constexpr int RBS = 4; /* row blocks of 16 per wave: a wave owns 64 rows of the tile */
    constexpr int SLOTS = NN + 1;
    float a[CB > 0 ? SLOTS : 1][CB > 0 ? CB : 1]; /* [slot][column block]: the lane's weight */
    nbc_v4u own_row = {0u, 0u, 0u, 0u}, halo_row = {0u, 0u, 0u, 0u};
    nbc_v4f bias4[CB > 0 ? CB : 1]; /* the lane's four output channels' biases, per column block */
    /* the frame's sampled rows 0..V, 16 bytes each; offsets beyond read zeros */
    auto sampled_rows = [&] {
        return __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(feat + (size_t) row_base * 4), 0, (int) min((uint64_t) (V + 1) * 16ull, 0xffffffffull), 0x00020000);
    };
    if constexpr (CB > 0) own_row = __builtin_amdgcn_raw_buffer_load_b128(sampled_rows(), (row0 + min((int) threadIdx.x, n_rows - 1)) * 16, 0, 0);

    const int cap = B.halo_cap;
    uint32_t* const tile_halo = B.tile_halo + (size_t) tile * VMHIP_HALO_MAX;
    uint32_t h_slot[MAX_ITEMS]; /* where the item's row went in the hash table */
#pragma unroll
    for (int k = 0; k < MAX_ITEMS; ++k) {
        const int out = outs[k];
        h_slot[k] = 0u;
        if (out >= 0 && (out < row0 || out >= row0 + VMHIP_TILE)) {
            uint32_t slot = hash((uint32_t) out);
            while (true) {
                const uint32_t prev = atomicCAS(&h_key[slot], EMPTY, (uint32_t) out);
                if (prev == EMPTY) { /* the row is new to the tile: it gets the next halo slot */
                    const int dense = atomicAdd(&halo_count, 1);
                    h_dense[slot] = (uint16_t) min(dense, 0xffff);
                    if (dense < cap) {
                        tile_halo[dense] = (uint32_t) row_base + (uint32_t) out;
                        if constexpr (CB > 0) halo_list[dense] = (uint32_t) out;
                    }
                    break;
                }
                if (prev == (uint32_t) out) break;
                slot = (slot + 1) & (NB_HASH - 1);
            }
            h_slot[k] = slot;
        }
    }
    __syncthreads();
    const int total = halo_count;
    if (threadIdx.x == 0) B.tile_desc[tile] = make_int4(row_base + row0, n_rows, min(total, cap), row_base);
    if constexpr (CB > 0) { /* the halo rows, one per thread, and the layer's weights */
        halo_row = __builtin_amdgcn_raw_buffer_load_b128(sampled_rows(), (int) threadIdx.x < min(total, cap) ? halo_list[threadIdx.x] * 16u : 0xffffffffu, 0, 0);
        const VM_GLOBAL float* const w = in_device_memory(reinterpret_cast<const float*>(L.w_mfma));
#pragma unroll
        for (int s = 0; s < SLOTS; ++s)
#pragma unroll
            for (int cb = 0; cb < CB; ++cb) a[s][cb] = w[(s * CB + cb) * 64 + (threadIdx.x & 63)];
        const VM_GLOBAL float* const bias = in_device_memory(L.b);
        const int q4 = ((threadIdx.x & 63) >> 4) * 4;
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) {
            bias4[cb] = nbc_v4f{0.0f, 0.0f, 0.0f, 0.0f};
            if (cb * 16 + q4 < L.c_out) bias4[cb] = *reinterpret_cast<const VM_GLOBAL nbc_v4f*>(bias + cb * 16 + q4); /* c_out is a multiple of 4 */
        }
    }

    typedef unsigned int row_words __attribute__((ext_vector_type(4)));
    uint16_t* const nbl_out = B.row_nbl + (size_t) row_base * VMHIP_NBL_STRIDE;
    auto position_of = [&](int out, uint32_t slot) {
        if (out >= row0 && out < row0 + VMHIP_TILE) return (uint32_t) (out - row0);
        const int dense = h_dense[slot];
        return dense < cap ? (uint32_t) (VMHIP_TILE + dense) : (uint32_t) VMHIP_NBL_FAR;
    };
    if constexpr (PER_ROW) {
        /* the row's entries packed two to a word (entries past nn are never read) */
        uint32_t words[4] = {0u, 0u, 0u, 0u};
#pragma unroll
        for (int k = 0; k < NN; ++k) words[k >> 1] |= (have_row ? position_of(outs[k], h_slot[k]) : 0u) << (16 * (k & 1));
        const row_words packed = {words[0], words[1], words[2], words[3]};
        if (have_row) write_element(reinterpret_cast<row_words*>(nbl_out), (Off) (row0 + threadIdx.x), packed);
        if constexpr (CB > 0) {
            *reinterpret_cast<row_words*>(nbl_rows[threadIdx.x]) = packed;
            __syncthreads();
        }
    }
    else {
#pragma unroll
        for (int k = 0; k < MAX_ITEMS; ++k) {
            const int out = outs[k];
            if (out >= 0) {
                /* the item's row of the tile and neighbour number, worked out again rather than kept in registers all the way */
                const int it = threadIdx.x + k * VMHIP_TILE;
                const int r = row_of(it);
                nbl_rows[r][it - r * nn] = (uint16_t) position_of(out, h_slot[k]);
            }
        }
        __syncthreads();
        /* one 16-byte store per row (entries past nn are never read) */
        if (have_row) write_element(reinterpret_cast<row_words*>(nbl_out), (Off) (row0 + threadIdx.x), *reinterpret_cast<const row_words*>(nbl_rows[threadIdx.x]));
    }

    /* ---- first layer, part two: contraction, activation, store ---- */
    if constexpr (CB > 0) {
        const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, q = lane >> 4, r16 = lane & 15;
        const int c_out = L.c_out, activation = L.activation;
        /* the rows the tile gathers, where the hash table was (every thread has passed the barrier after its last look at it) */
        nbc_v4u* const staged = reinterpret_cast<nbc_v4u*>(h_key);
        staged[threadIdx.x] = own_row;
        staged[VMHIP_TILE + threadIdx.x] = halo_row;
        __syncthreads();
        const float* const staged_f = reinterpret_cast<const float*>(h_key);
        float x[RBS][SLOTS]; /* [row block][slot]: the lane's channel of the slot's source row */
        /* block-uniform: every halo row of the tile has a slot (nearly always). The code is compiled for both cases,
         * so that the usual one carries no test per position. */
        const bool all_staged = total <= cap;
        auto gather = [&](auto checked_tag) {
            constexpr bool CHECKED = decltype(checked_tag)::value;
#pragma unroll
            for (int rb = 0; rb < RBS; ++rb) {
                const int row_t = min(wave * 64 + rb * 16 + r16, n_rows - 1); /* lanes past the tile's rows repeat its last row and store nothing */
                const nbc_v4u positions = *reinterpret_cast<const nbc_v4u*>(nbl_rows[row_t]);
                x[rb][0] = staged_f[row_t * 4 + q];
#pragma unroll
                for (int s = 0; s < NN; ++s) {
                    const uint32_t word = (s >> 1) == 0 ? positions.x : (s >> 1) == 1 ? positions.y : (s >> 1) == 2 ? positions.z : positions.w;
                    const uint32_t at = (s & 1) ? (word >> 16) : (word & 0xffffu);
                    /* a position that is not staged reads slot 0 here and is patched below */
                    x[rb][s + 1] = staged_f[(CHECKED && at == VMHIP_NBL_FAR ? 0u : at) * 4 + q];
                }
            }
        };
        if (all_staged) gather(std::false_type());
        else gather(std::true_type());
        if (!all_staged) { /* more halo rows than slots: those rows' numbers from the table this block has just written */
#pragma unroll
            for (int rb = 0; rb < RBS; ++rb) {
                const int row_t = min(wave * 64 + rb * 16 + r16, n_rows - 1);
#pragma unroll
                for (int s = 0; s < NN; ++s) {
                    if (nbl_rows[row_t][s] == VMHIP_NBL_FAR) {
                        const int g = read_element(nb_out, (Off) (row0 + row_t) * nb_stride + (Off) s);
                        x[rb][s + 1] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(sampled_rows(), g * 16 + q * 4, 0, 0));
                    }
                }
            }
        }
        nbc_v4f acc[RBS][CB];
#pragma unroll
        for (int cb = 0; cb < CB; ++cb)
#pragma unroll
            for (int rb = 0; rb < RBS; ++rb) acc[rb][cb] = bias4[cb];
#pragma unroll
        for (int s = 0; s < SLOTS; ++s)
#pragma unroll
            for (int cb = 0; cb < CB; ++cb)
#pragma unroll
                for (int rb = 0; rb < RBS; ++rb) acc[rb][cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[s][cb], x[rb][s], acc[rb][cb], 0, 0, 0);
        /* one uniform branch for all the values */
        auto for_each_value = [&](auto fn) {
#pragma unroll
            for (int rb = 0; rb < RBS; ++rb)
#pragma unroll
                for (int cb = 0; cb < CB; ++cb)
#pragma unroll
                    for (int v = 0; v < 4; ++v) acc[rb][cb][v] = fn(acc[rb][cb][v]);
        };
        if (activation == VMHIP_SELU) for_each_value([](float t) { return nbc_selu(t); });
        else if (activation == VMHIP_RELU) for_each_value([](float t) { return fmaxf(t, 0.0f); });
        else for_each_value([](float t) { return tanhf(t); });
        /* the tile's output rows; a lane without a row, or a column block's padding, gets an offset the hardware drops */
        const __amdgpu_buffer_rsrc_t out_rsrc =
          __builtin_amdgcn_make_buffer_rsrc(layer_out + ((size_t) row_base + row0) * c_out, 0, VMHIP_TILE * c_out * 4, 0x00020000);
#pragma unroll
        for (int rb = 0; rb < RBS; ++rb) {
            const int row_t = wave * 64 + rb * 16 + r16;
#pragma unroll
            for (int cb = 0; cb < CB; ++cb) {
                const int o = cb * 16 + q * 4;
                __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(nbc_v4u, acc[rb][cb]), out_rsrc,
                                                       (row_t < n_rows && o < c_out) ? (uint32_t) (row_t * c_out + o) * 4u : 0xffffffffu, 0, 0);
            }
        }
    }
}

}  // namespace

void vm_launch_libm(int which, const float* x, float* y, int n, hipStream_t stream) {
    hipLaunchKernelGGL(vm_libm_kernel, dim3((n + 255) / 256), dim3(256), 0, stream, which, x, y, n);
}
void vm_launch_copy_probe(const void* src, void* dst, size_t bytes, hipStream_t stream) {
    const size_t n = bytes / 16;
    hipLaunchKernelGGL(vm_copy_probe_kernel, dim3(256 * 16), dim3(256), 0, stream, reinterpret_cast<const float4*>(src),
                       reinterpret_cast<float4*>(dst), n);
}
void vm_launch_stream_probe(const void* src, void* dst, size_t rows, int read_bytes_per_row, int write_bytes_per_row, hipStream_t stream) {
    hipLaunchKernelGGL(vm_stream_probe_kernel, dim3(256 * 16), dim3(256), 0, stream, reinterpret_cast<const uint4*>(src), reinterpret_cast<uint4*>(dst),
                       rows / 64, read_bytes_per_row * 4, write_bytes_per_row * 4);
}
void vm_launch_publish(int32_t* counts, int n_counts, const int2* amb_list, int amb_stride, int amb_head, int n_frames, const unsigned int* timeouts, uint32_t* epoch,
                       int32_t* host_counts, int2* host_amb, uint32_t* host_timeouts, hipStream_t stream) {
    hipLaunchKernelGGL(vm_publish_kernel, dim3(n_frames > 0 ? n_frames : 1), dim3(64), 0, stream, counts, n_counts, amb_list, amb_stride, amb_head, timeouts, epoch,
                       host_counts, host_amb, host_timeouts);
}
void vm_launch_project(const VmBatchDev& B, hipStream_t stream) {
    if (B.n_cand_tiles > 0) hipLaunchKernelGGL(vm_project_kernel, dim3(B.n_cand_tiles), dim3(VMHIP_TILE), 0, stream, B);
}
void vm_launch_compact(const VmBatchDev& B, float* feat, int classify, hipStream_t stream) {
    if (B.n_cand_tiles > 0)
        hipLaunchKernelGGL(vm_compact_kernel, dim3(B.n_cand_tiles), dim3(VMHIP_TILE), 0, stream, B,
                           reinterpret_cast<float4*>(feat), classify);
}
void vm_launch_lookup_export(const VmBatchDev& B, int same_edges, float* vectors, int32_t* graph, float* pixels, hipStream_t stream) {
    if (B.n_cand_tiles > 0)
        hipLaunchKernelGGL(vm_lookup_export_kernel, dim3(B.n_cand_tiles), dim3(VMHIP_TILE), 0, stream, B, same_edges, vectors, graph,
                           reinterpret_cast<float2*>(pixels));
}

void vm_launch_lookup(const VmLookupFrame* frames, int n_frames, hipStream_t stream) {
    if (n_frames > 0) hipLaunchKernelGGL(vm_lookup_kernel, dim3(n_frames), dim3(LOOKUP_THREADS), 0, stream, frames);
}

template <bool WIDE>
static void launch_neighbourhood(const VmBatchDev& B, hipStream_t stream) {
    const dim3 grid(B.n_row_tiles), block(VMHIP_TILE);
    const VmLayerDev none{};
    switch (B.uniform_nn) {
        case 4: hipLaunchKernelGGL((vm_neighbourhood_kernel<WIDE, 4, 0>), grid, block, 0, stream, B, none, nullptr, nullptr); break;
        case 6: hipLaunchKernelGGL((vm_neighbourhood_kernel<WIDE, 6, 0>), grid, block, 0, stream, B, none, nullptr, nullptr); break;
        case 8: hipLaunchKernelGGL((vm_neighbourhood_kernel<WIDE, 8, 0>), grid, block, 0, stream, B, none, nullptr, nullptr); break;
        default: hipLaunchKernelGGL((vm_neighbourhood_kernel<WIDE, 0, 0>), grid, block, 0, stream, B, none, nullptr, nullptr); break;
    }
}
void vm_launch_neighbourhood(const VmBatchDev& B, hipStream_t stream) {
    if (B.n_row_tiles <= 0) return;
    if (B.wide_offsets) launch_neighbourhood<true>(B, stream);
    else launch_neighbourhood<false>(B, stream);
}

bool vm_neighbourhood_conv_supported(int c_in, int c_out, int slots, int activation) {
    return c_in == 4 && c_out >= 4 && c_out <= 32 && c_out % 4 == 0 && (slots == 5 || slots == 7 || slots == 9) && activation != VMHIP_SOFTMAX;
}
template <bool WIDE, int NN>
static void launch_neighbourhood_conv(const VmBatchDev& B, const VmLayerDev& L, const float* in, float* out, hipStream_t stream) {
    const dim3 grid(B.n_row_tiles), block(VMHIP_TILE);
    if (L.c_out <= 16) hipLaunchKernelGGL((vm_neighbourhood_kernel<WIDE, NN, 1>), grid, block, 0, stream, B, L, in, out);
    else hipLaunchKernelGGL((vm_neighbourhood_kernel<WIDE, NN, 2>), grid, block, 0, stream, B, L, in, out);
}
int vm_launch_neighbourhood_conv(const VmBatchDev& B, const VmLayerDev& L, const float* in, float* out, hipStream_t stream, const char** kernel_name) {
    if (!vm_neighbourhood_conv_supported(L.c_in, L.c_out, L.slots, L.activation) || !B.row_nbl || !L.w_mfma || !L.b || L.in_bf16 || L.out_bf16 || L.arith_bf16
        || B.uniform_nn != L.slots - 1)
        return -1;
    if (kernel_name) *kernel_name = vm_kernel_name("neighbourhood_conv", L.c_in, L.c_out, L.slots);
    if (B.n_row_tiles <= 0) return 0;
#define X(NN)                                                                             \
    case NN:                                                                              \
        if (B.wide_offsets) launch_neighbourhood_conv<true, NN>(B, L, in, out, stream);   \
        else launch_neighbourhood_conv<false, NN>(B, L, in, out, stream);                 \
        break;
    switch (B.uniform_nn) {
        X(4)
        X(6)
        X(8)
        default: return -1;
    }
#undef X
    return 0;
}

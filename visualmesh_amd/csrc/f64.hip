/*
 * f64.hip - the engine for Scalar = double: the entry points of include/visualmesh_hip.h that end in _f64.
 *
 * The reference's engines are templates over Scalar (engine/cpu/engine.hpp:49-50); this file is the double
 * instantiation of the same path - projection of every candidate, the strict on-screen filter, order-preserving
 * compaction, the neighbourhood table, sampling, and per layer gather + dense + activation - with every stage in fp64
 * on the device. It serves callers that need the reference's double results (a training bridge, checks of the float
 * path), not throughput: one frame per call, plain kernels for the memory-bound stages, and the layers on the fp64
 * matrix instruction v_mfma_f64_16x16x4_f64 (one wave = 16 rows x up to 128 outputs, operands straight from global
 * memory, no LDS and no barrier, so any layer shape takes the same kernel).
 *
 * The device's acos/sin/tan/sqrt differ from the host C library's in the last bits, so, as in the float path, a
 * candidate that projects within a narrow band of a screen edge is listed and decided again on the host with the
 * reference's own expression order (host_project.cpp). The band is 1e-6 px: about 1e6 times the difference it guards.
 */
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstring>
#include <string>
#include <vector>

#include "host_project.h"
#include "visualmesh_hip.h"
#include "vmhip_internal.h"

namespace {

constexpr int F64_BLOCK = 256;
constexpr int F64_NEAR_CAP = 8192;      /* listed near-edge candidates per frame before the host takes all of them */
constexpr double F64_BAND = 1.0e-6;     /* px */
constexpr int F64_MAX_SOFTMAX = 128;

int fail64(int code, const std::string& msg) { return vm_set_error(code, msg.c_str()); }
#define HIP_TRY64(expr)                                                                              \
    do {                                                                                             \
        hipError_t e_ = (expr);                                                                      \
        if (e_ != hipSuccess)                                                                        \
            return fail64(VMHIP_ERR_HIP, std::string(#expr) + " failed: " + hipGetErrorString(e_)); \
    } while (0)

struct Frame64 {
    const double* rays;
    const int32_t* mesh_nbr;
    int32_t n_nodes, nn;
    double Rco[9];
    int32_t projection;
    double focal, centre[2], ik[4];
    int32_t width, height;
    const int32_t* range_first;   /* [n_ranges] */
    const int32_t* range_prefix;  /* [n_ranges + 1] candidates before each range */
    int32_t n_ranges, n_cand;
    const uint8_t* image;
    int32_t fmt;
    double band, px_error;
};

/* everything a pass writes; V = counters[0] once the scan has run, counters[1] = listed near-edge candidates */
struct Work64 {
    double2* cand_px;      /* [n_cand] */
    uint8_t* keep;         /* [n_cand] */
    int32_t* near;         /* [F64_NEAR_CAP] candidate slots */
    int32_t* counters;     /* [4] */
    int32_t* block_count;  /* [blocks] kept candidates per block, then their exclusive prefix */
    double2* row_px;       /* [n_cand] */
    int32_t* gidx;         /* [n_cand] */
    int32_t* r_lookup;     /* [n_nodes + 1] row of a node, -1 = not visible */
    int32_t* nb;           /* [n_cand + 1][nn] */
};

__device__ __forceinline__ int cand_to_node(const Frame64& F, int p) {
    int lo = 0, hi = F.n_ranges - 1;
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (F.range_prefix[mid] <= p) lo = mid;
        else hi = mid - 1;
    }
    return F.range_first[lo] + (p - F.range_prefix[lo]);
}

/* reference utility/projection.hpp:162-187 for Scalar = double, dot order of utility/math.hpp:145-164 */
__device__ __forceinline__ double2 project64(const Frame64& F, double rx, double ry, double rz) {
    const double c0 = F.Rco[2] * rz + (F.Rco[1] * ry + F.Rco[0] * rx);
    const double c1 = F.Rco[5] * rz + (F.Rco[4] * ry + F.Rco[3] * rx);
    const double c2 = F.Rco[8] * rz + (F.Rco[7] * ry + F.Rco[6] * rx);
    const double theta = acos(c0);
    const double rsin_theta = 1.0 / sqrt(1.0 - c0 * c0);
    double r_u;
    if (F.projection == VMHIP_RECTILINEAR) r_u = F.focal * tan(fmin(fmax(theta, 0.0), 1.57079632679489661923));
    else if (F.projection == VMHIP_EQUISOLID) r_u = 2.0 * F.focal * sin(theta * 0.5);
    else r_u = F.focal * theta;
    const double r2 = r_u * r_u;
    const double s = 1.0 + F.ik[0] * r2 + F.ik[1] * (r2 * r2) + F.ik[2] * (r2 * r2) * r2 + F.ik[3] * (r2 * r2) * (r2 * r2);
    const double r_d = r_u * s;
    double sx = 0.0, sy = 0.0;
    if (!(c0 >= 1.0)) {
        sx = r_d * c1 * rsin_theta;
        sy = r_d * c2 * rsin_theta;
    }
    double2 px;
    px.x = ((double) F.width * 0.5 - sx) - F.centre[0] + F.px_error;
    px.y = ((double) F.height * 0.5 - sy) - F.centre[1] + F.px_error;
    return px;
}

__global__ __launch_bounds__(F64_BLOCK) void f64_fill_kernel(int32_t* p, int n, int32_t v, int32_t* counters) {
    const int i = blockIdx.x * F64_BLOCK + threadIdx.x;
    if (i < n) p[i] = v;
    if (i < 4) counters[i] = 0;
}

/* engine/cpu/engine.hpp:97-125: project, strict on-screen test; candidates near an edge are listed for the host */
__global__ __launch_bounds__(F64_BLOCK) void f64_project_kernel(Frame64 F, Work64 W) {
    const int p = blockIdx.x * F64_BLOCK + threadIdx.x;
    if (p >= F.n_cand) return;
    const int node = cand_to_node(F, p);
    const double2 px = project64(F, F.rays[3 * (size_t) node], F.rays[3 * (size_t) node + 1], F.rays[3 * (size_t) node + 2]);
    const double w = (double) F.width, h = (double) F.height;
    const bool keep = 0.0 <= px.x && px.x + 1.0 < w && 0.0 <= px.y && px.y + 1.0 < h;
    /* NaN pixels fail every comparison on host and device alike and are never near */
    const bool near = fabs(px.x) < F.band || fabs(px.x + 1.0 - w) < F.band || fabs(px.y) < F.band || fabs(px.y + 1.0 - h) < F.band;
    W.cand_px[p] = px;
    W.keep[p] = keep ? 1 : 0;
    if (near) {
        const int slot = atomicAdd(&W.counters[1], 1);
        if (slot < F64_NEAR_CAP) W.near[slot] = p;
    }
}

__device__ __forceinline__ int block_exclusive_scan(int v, int* wave_totals, int& total) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int incl = v;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const int o = __shfl_up(incl, d, 64);
        if (lane >= d) incl += o;
    }
    if (lane == 63) wave_totals[wave] = incl;
    __syncthreads();
    int before = 0;
    total = 0;
#pragma unroll
    for (int w = 0; w < F64_BLOCK / 64; ++w) {
        if (w < wave) before += wave_totals[w];
        total += wave_totals[w];
    }
    __syncthreads();
    return before + incl - v;
}

__global__ __launch_bounds__(F64_BLOCK) void f64_count_kernel(Frame64 F, Work64 W) {
    __shared__ int wave_totals[F64_BLOCK / 64];
    const int p = blockIdx.x * F64_BLOCK + threadIdx.x;
    const int k = p < F.n_cand ? W.keep[p] : 0;
    int total;
    block_exclusive_scan(k, wave_totals, total);
    if (threadIdx.x == 0) W.block_count[blockIdx.x] = total;
}

/* one block: exclusive prefix of the block counts in place, the total = number of visible nodes */
__global__ __launch_bounds__(F64_BLOCK) void f64_scan_kernel(Work64 W, int n_blocks) {
    __shared__ int wave_totals[F64_BLOCK / 64];
    int carry = 0;
    for (int base = 0; base < n_blocks; base += F64_BLOCK) {
        const int i = base + threadIdx.x;
        const int v = i < n_blocks ? W.block_count[i] : 0;
        int total;
        const int before = block_exclusive_scan(v, wave_totals, total);
        if (i < n_blocks) W.block_count[i] = carry + before;
        carry += total;
    }
    if (threadIdx.x == 0) W.counters[0] = carry;
}

__global__ __launch_bounds__(F64_BLOCK) void f64_scatter_kernel(Frame64 F, Work64 W) {
    __shared__ int wave_totals[F64_BLOCK / 64];
    const int p = blockIdx.x * F64_BLOCK + threadIdx.x;
    const int k = p < F.n_cand ? W.keep[p] : 0;
    int total;
    const int before = block_exclusive_scan(k, wave_totals, total);
    if (k) {
        const int row = W.block_count[blockIdx.x] + before;
        const int node = cand_to_node(F, p);
        W.row_px[row] = W.cand_px[p];
        W.gidx[row] = node;
        W.r_lookup[node] = row;
    }
}

/* engine/cpu/engine.hpp:127-143: local neighbour table through the reverse lookup, the null row last */
__global__ __launch_bounds__(F64_BLOCK) void f64_neighbourhood_kernel(Frame64 F, Work64 W) {
    const int V = W.counters[0];
    const int i = blockIdx.x * F64_BLOCK + threadIdx.x;
    const int row = i / F.nn, t = i - row * F.nn;
    if (row > V) return;
    int v = V;
    if (row < V) {
        const int r = W.r_lookup[F.mesh_nbr[(size_t) W.gidx[row] * F.nn + t]];
        v = r < 0 ? V : r;
    }
    W.nb[(size_t) row * F.nn + t] = v;
}

/* ---- sampling: engine/cpu/pixel.hpp:43-144 and bayer.hpp:95-158 for Scalar = double ---- */
struct d4 {
    double x, y, z, w;
};
#define INV255_64 (1.0 / 255.0)

__device__ __forceinline__ d4 texel64(const Frame64& F, int x, int y) {
    const size_t idx = (size_t) y * F.width + x;
    d4 o;
    switch (F.fmt) {
        case VMHIP_FMT_RGBA: {
            const uint8_t* b = F.image + idx * 4;
            o = d4{b[0] * INV255_64, b[1] * INV255_64, b[2] * INV255_64, b[3] * INV255_64};
        } break;
        case VMHIP_FMT_BGRA: {
            const uint8_t* b = F.image + idx * 4;
            o = d4{b[2] * INV255_64, b[1] * INV255_64, b[0] * INV255_64, b[3] * INV255_64};
        } break;
        case VMHIP_FMT_RGB3: {
            const uint8_t* b = F.image + idx * 3;
            o = d4{b[0] * INV255_64, b[1] * INV255_64, b[2] * INV255_64, 1.0};
        } break;
        case VMHIP_FMT_BGR3: {
            const uint8_t* b = F.image + idx * 3;
            o = d4{b[2] * INV255_64, b[1] * INV255_64, b[0] * INV255_64, 1.0};
        } break;
        default: {
            const double v = F.image[idx] * INV255_64;
            o = d4{v, v, v, 1.0};
        } break;
    }
    return o;
}

__device__ __forceinline__ int bayer_raw(const Frame64& F, int x, int y) {
    const int xc = min(max(x, 0), F.width - 1), yc = min(max(y, 0), F.height - 1);
    return F.image[(size_t) yc * F.width + xc];
}
/* which colour site (x, y) is: 0 R, 1 G on a red row, 2 G on a blue row, 3 B (bayer.hpp:140-155) */
__device__ __forceinline__ int bayer_site(int fmt, int x, int y) {
    const int i = ((y & 1) << 1) | (x & 1);
    switch (fmt) {
        case VMHIP_FMT_GRBG: return (0x2301 >> (i * 4)) & 0xf;
        case VMHIP_FMT_RGGB: return (0x3210 >> (i * 4)) & 0xf;
        case VMHIP_FMT_GBRG: return (0x1032 >> (i * 4)) & 0xf;
        default: return (0x0123 >> (i * 4)) & 0xf;
    }
}
/* Malvar-He-Cutler on the 5x5 patch around (x, y), borders clamped; integer arithmetic, truncating division by 64, no
 * clamp of the result (bayer.hpp:95-108) */
__device__ d4 demosaic64(const Frame64& F, int x, int y) {
#define P(r, c) bayer_raw(F, x - 2 + (c), y - 2 + (r))
    const int site = bayer_site(F.fmt, x, y);
    const int centre = P(2, 2);
    int red, green, blue;
    if (site == 0 || site == 3) {
        const int arms = P(0, 2) + P(2, 0) + P(2, 4) + P(4, 2);
        const int cross = (-8 * arms + 16 * (P(1, 2) + P(2, 1) + P(2, 3) + P(3, 2)) + 32 * centre) / 64;
        const int checker = (-12 * arms + 16 * (P(1, 1) + P(1, 3) + P(3, 1) + P(3, 3)) + 48 * centre) / 64;
        green = cross;
        red = site == 0 ? centre : checker;
        blue = site == 0 ? checker : centre;
    }
    else {
        const int diag = P(1, 1) + P(1, 3) + P(3, 1) + P(3, 3);
        const int horiz = (4 * (P(0, 2) + P(4, 2)) - 8 * diag - 8 * (P(2, 0) + P(2, 4)) + 32 * (P(2, 1) + P(2, 3)) + 40 * centre) / 64;
        const int vert = (-8 * (P(0, 2) + P(4, 2)) - 8 * diag + 32 * (P(1, 2) + P(3, 2)) + 4 * (P(2, 0) + P(2, 4)) + 40 * centre) / 64;
        green = centre;
        red = site == 1 ? horiz : vert;
        blue = site == 1 ? vert : horiz;
    }
#undef P
    return d4{red * INV255_64, green * INV255_64, blue * INV255_64, 255 * INV255_64};
}

/* rows 0..V-1: bilinear sample at the node's pixel; row V: the null row (-1, -1, -1, -1) (engine.hpp:198-206) */
__global__ __launch_bounds__(F64_BLOCK) void f64_sample_kernel(Frame64 F, Work64 W, double* __restrict__ feat) {
    const int V = W.counters[0];
    const int row = blockIdx.x * F64_BLOCK + threadIdx.x;
    if (row > V) return;
    d4 o{-1.0, -1.0, -1.0, -1.0};
    if (row < V) {
        const double2 px = W.row_px[row];
        const int x1 = max((int) floor(px.x), 0), y1 = max((int) floor(px.y), 0);
        const int x2 = min(x1 + 1, F.width - 1), y2 = min(y1 + 1, F.height - 1);
        const bool bayer = F.fmt >= VMHIP_FMT_GRBG && F.fmt <= VMHIP_FMT_BGGR;
        const d4 q1 = bayer ? demosaic64(F, x1, y1) : texel64(F, x1, y1);
        const d4 q2 = bayer ? demosaic64(F, x2, y1) : texel64(F, x2, y1);
        const d4 q3 = bayer ? demosaic64(F, x1, y2) : texel64(F, x1, y2);
        const d4 q4 = bayer ? demosaic64(F, x2, y2) : texel64(F, x2, y2);
        const double wxa = ((double) x2 - px.x) / (double) (x2 - x1), wxb = (px.x - (double) x1) / (double) (x2 - x1);
        const double wya = ((double) y2 - px.y) / (double) (y2 - y1), wyb = (px.y - (double) y1) / (double) (y2 - y1);
        o.x = (q1.x * wxa + q2.x * wxb) * wya + (q3.x * wxa + q4.x * wxb) * wyb;
        o.y = (q1.y * wxa + q2.y * wxb) * wya + (q3.y * wxa + q4.y * wxb) * wyb;
        o.z = (q1.z * wxa + q2.z * wxb) * wya + (q3.z * wxa + q4.z * wxb) * wyb;
        o.w = (q1.w * wxa + q2.w * wxb) * wya + (q3.w * wxa + q4.w * wxb) * wyb;
    }
    double* f = feat + (size_t) row * 4;
    f[0] = o.x, f[1] = o.y, f[2] = o.z, f[3] = o.w;
}

/* ---- one layer: gather [self, neighbours] (slots > 1) or the row itself, dense, activation -------------------------
 * v_mfma_f64_16x16x4_f64: A is 16 rows x 4 inputs (lane l holds row l % 16, input l / 16), B is 4 inputs x 16 outputs
 * (lane l holds input l / 16, output l % 16), D is 16 x 16 (the four values of lane l are rows l / 16 + 0, 4, 8, 12 of
 * output l % 16: the rows of a lane are interleaved, unlike the fp32 instruction's four consecutive rows).
 * A wave owns 16 rows and walks the outputs in groups of NT tiles of 16; weights are padded with zeros to whole tiles
 * ([slots * c_in_pad][n_pad], c_in_pad a multiple of 4, n_pad of 16), inputs past c_in are read as zero. */
typedef double v4d __attribute__((ext_vector_type(4)));

struct Layer64 {
    const double* w;  /* padded weights */
    const double* b;  /* [n_pad] */
    int32_t c_in, c_in_pad, n_out, n_pad, slots, activation;
};

__device__ __forceinline__ double activate64(int act, double v) {
    switch (act) {
        case VMHIP_SELU: return 1.0507009873554804934193349852946 * (v >= 0.0 ? v : 1.6732632423543772848170429916717 * exp(v) - 1.6732632423543772848170429916717);
        case VMHIP_RELU: return fmax(v, 0.0);
        case VMHIP_TANH: return tanh(v);
        default: return exp(v); /* softmax: the division follows */
    }
}

template <int NT>
__global__ __launch_bounds__(F64_BLOCK) void f64_layer_kernel(Layer64 L, const int32_t* __restrict__ counters, const int32_t* __restrict__ nb,
                                                             int nn, const double* __restrict__ in, double* __restrict__ out) {
    const int V = counters[0];
    const int rows = V + 1;
    const int lane = threadIdx.x & 63;
    const int row0 = (blockIdx.x * (F64_BLOCK / 64) + (threadIdx.x >> 6)) * 16;
    if (row0 >= rows) return;
    const int a_row = row0 + (lane & 15);  /* the row this lane feeds into A */
    const int kk = lane >> 4;              /* and which of the 4 inputs of a step */
    const int col = lane & 15;
    const bool a_live = a_row < rows;

    for (int group = 0; group * NT * 16 < L.n_pad; ++group) {
        const int col0 = group * NT * 16;
        v4d acc[NT];
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            const double bias = col0 + t * 16 < L.n_pad ? L.b[col0 + t * 16 + col] : 0.0;
            acc[t] = v4d{bias, bias, bias, bias};
        }
        for (int s = 0; s < L.slots; ++s) {
            int src = a_live ? a_row : 0;
            if (s > 0 && a_live) src = nb[(size_t) a_row * nn + (s - 1)];
            const double* a_ptr = in + (size_t) src * L.c_in;
            const double* w_ptr = L.w + (size_t) s * L.c_in_pad * L.n_pad + col0 + col;
            for (int c = 0; c < L.c_in_pad; c += 4) {
                const double a = (a_live && c + kk < L.c_in) ? a_ptr[c + kk] : 0.0;
#pragma unroll
                for (int t = 0; t < NT; ++t) {
                    if (col0 + t * 16 < L.n_pad) {
                        const double b = w_ptr[(size_t) (c + kk) * L.n_pad + t * 16];
                        acc[t] = __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, acc[t], 0, 0, 0);
                    }
                }
            }
        }
        /* activation; a softmax layer fits one group (checked on the host): a row's sum runs over the 16 lanes that hold
         * it and over the tiles */
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[t][r] = activate64(L.activation, acc[t][r]);
        if (L.activation == VMHIP_SOFTMAX) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                double sum = 0.0;
#pragma unroll
                for (int t = 0; t < NT; ++t)
                    if (col0 + t * 16 + col < L.n_out) sum += acc[t][r];
#pragma unroll
                for (int d = 1; d < 16; d <<= 1) sum += __shfl_xor(sum, d, 64);
#pragma unroll
                for (int t = 0; t < NT; ++t) acc[t][r] = acc[t][r] / sum;
            }
        }
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            const int c = col0 + t * 16 + col;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int row = row0 + 4 * r + (lane >> 4);
                if (c < L.n_out && row < rows) out[(size_t) row * L.n_out + c] = acc[t][r];
            }
        }
    }
}

struct Buf64 {
    void* p = nullptr;
    size_t cap = 0;
    int ensure(size_t bytes) {
        if (bytes <= cap) return VMHIP_OK;
        if (p) (void) hipFree(p);
        p = nullptr, cap = 0;
        const size_t want = bytes + bytes / 4 + 256;
        if (hipMalloc(&p, want) != hipSuccess) return VMHIP_ERR_HIP;
        cap = want;
        return VMHIP_OK;
    }
    void release() {
        if (p) (void) hipFree(p);
        p = nullptr, cap = 0;
    }
};

struct HostLayer64 {
    Layer64 dev{};
    double *d_w = nullptr, *d_b = nullptr;
};

}  // namespace

struct vmhip_mesh_f64 {
    double* d_rays = nullptr;
    int32_t* d_nbr = nullptr;
    std::vector<double> h_rays;  /* the host's copy: near-edge candidates are decided again from it */
    int32_t n_nodes = 0, nn = 0;
};

struct vmhip_engine_f64 {
    int32_t nn = 0, n_classes = 4, max_width = 4;
    std::vector<HostLayer64> layers;
    hipStream_t stream = nullptr;
    Buf64 ranges, cand_px, keep, near, counters, block_count, row_px, gidx, r_lookup, nb, feat_a, feat_b, image;
    int64_t listed = 0, overruled = 0;
};

namespace {

void launch_layer(const Layer64& L, const int32_t* counters, const int32_t* nb, int nn, const double* in, double* out, int max_rows,
                  hipStream_t stream) {
    const int waves = (max_rows + 15) / 16;
    const dim3 grid((waves + F64_BLOCK / 64 - 1) / (F64_BLOCK / 64)), block(F64_BLOCK);
    const int tiles = L.n_pad / 16;
    if (tiles <= 1) hipLaunchKernelGGL(f64_layer_kernel<1>, grid, block, 0, stream, L, counters, nb, nn, in, out);
    else if (tiles <= 2) hipLaunchKernelGGL(f64_layer_kernel<2>, grid, block, 0, stream, L, counters, nb, nn, in, out);
    else if (tiles <= 4) hipLaunchKernelGGL(f64_layer_kernel<4>, grid, block, 0, stream, L, counters, nb, nn, in, out);
    else hipLaunchKernelGGL(f64_layer_kernel<8>, grid, block, 0, stream, L, counters, nb, nn, in, out);
}

int run64(vmhip_engine_f64* E, const vmhip_frame_f64* in, vmhip_result_f64* out, bool classify) {
    if (!E || !in || !out) return fail64(VMHIP_ERR_ARGUMENT, "f64: null argument");
    const vmhip_mesh_f64* M = in->mesh;
    if (!M) return fail64(VMHIP_ERR_ARGUMENT, "f64: frame without a mesh");
    if (in->lens.projection < VMHIP_RECTILINEAR || in->lens.projection > VMHIP_EQUIDISTANT)
        return fail64(VMHIP_ERR_LENS, "Cannot project: Unknown lens type");
    if (in->lens.width <= 0 || in->lens.height <= 0) return fail64(VMHIP_ERR_ARGUMENT, "f64: empty image dimensions");
    if (in->n_ranges < 0 || (in->n_ranges > 0 && !in->ranges)) return fail64(VMHIP_ERR_ARGUMENT, "f64: bad range table");
    if (classify && !E->layers.empty() && M->nn != E->nn)
        return fail64(VMHIP_ERR_ARGUMENT, "f64: the mesh's neighbour count does not match the network");
    int fmt = VMHIP_FMT_NONE, bpp = 0;
    if (classify) {
        if (!vm_decode_fourcc(in->fourcc, &fmt, &bpp)) {
            const uint32_t f = in->fourcc;
            const char text[5] = {char(f & 0xff), char((f >> 8) & 0xff), char((f >> 16) & 0xff), char((f >> 24) & 0xff), 0};
            return fail64(VMHIP_ERR_FORMAT, std::string("Unsupported image format ") + text);
        }
        if (!in->image) return fail64(VMHIP_ERR_ARGUMENT, "f64: classification needs an image");
    }
    out->n_visible = 0;

    /* ranges -> first[] and prefix[] */
    const int nr = in->n_ranges;
    std::vector<int32_t> table(size_t(2) * nr + 1);
    int64_t total = 0;
    int32_t last_end = 0;
    for (int r = 0; r < nr; ++r) {
        const int32_t a = in->ranges[2 * r], e = in->ranges[2 * r + 1];
        if (a < last_end || e < a || e > M->n_nodes) return fail64(VMHIP_ERR_ARGUMENT, "f64: ranges must be ascending, disjoint and inside the mesh");
        table[r] = a;
        table[size_t(nr) + r] = int32_t(total);
        total += e - a;
        last_end = e;
    }
    table[size_t(2) * nr] = int32_t(total);
    if (total > 0x7fff0000) return fail64(VMHIP_ERR_ARGUMENT, "f64: too many candidates");
    if (total == 0) return VMHIP_OK;
    const int n_cand = int(total);
    if (out->capacity < n_cand) return fail64(VMHIP_ERR_CAPACITY, "f64: result capacity is smaller than the number of candidates");

    const int n_blocks = (n_cand + F64_BLOCK - 1) / F64_BLOCK;
    const size_t rows = size_t(n_cand) + 1;
    const size_t image_bytes = classify ? size_t(in->lens.width) * in->lens.height * bpp : 0;
    if (E->ranges.ensure(table.size() * 4) || E->cand_px.ensure(size_t(n_cand) * 16) || E->keep.ensure(n_cand) || E->near.ensure(F64_NEAR_CAP * 4)
        || E->counters.ensure(16) || E->block_count.ensure(size_t(n_blocks) * 4) || E->row_px.ensure(size_t(n_cand) * 16)
        || E->gidx.ensure(size_t(n_cand) * 4) || E->r_lookup.ensure((size_t(M->n_nodes) + 1) * 4) || E->nb.ensure(rows * std::max(M->nn, 1) * 4)
        || (classify && (E->feat_a.ensure(rows * E->max_width * 8) || E->feat_b.ensure(rows * E->max_width * 8) || E->image.ensure(image_bytes))))
        return fail64(VMHIP_ERR_HIP, "f64: out of device memory");

    hipStream_t s = E->stream;
    HIP_TRY64(hipMemcpyAsync(E->ranges.p, table.data(), table.size() * 4, hipMemcpyHostToDevice, s));
    if (classify) HIP_TRY64(hipMemcpyAsync(E->image.p, in->image, image_bytes, hipMemcpyHostToDevice, s));

    Frame64 F;
    std::memset(&F, 0, sizeof(F));
    F.rays = M->d_rays, F.mesh_nbr = M->d_nbr, F.n_nodes = M->n_nodes, F.nn = M->nn;
    std::memcpy(F.Rco, in->Rco, sizeof(F.Rco));
    F.projection = in->lens.projection;
    F.focal = in->lens.focal_length;
    F.centre[0] = in->lens.centre[0], F.centre[1] = in->lens.centre[1];
    vm_host_inverse_coefficients_f64(in->lens.k, F.ik);
    F.width = in->lens.width, F.height = in->lens.height;
    F.range_first = static_cast<const int32_t*>(E->ranges.p);
    F.range_prefix = F.range_first + nr;
    F.n_ranges = nr, F.n_cand = n_cand;
    F.image = static_cast<const uint8_t*>(E->image.p);
    F.fmt = fmt;
    double band = 0.0, px_error = 0.0;
    vm_debug_knobs(&px_error, &band);
    /* the float path's default band is its own; only a band set by a test carries over */
    F.band = band != double(VMHIP_AMB_EPS_DEFAULT) ? band : F64_BAND;
    F.px_error = px_error;

    Work64 W;
    W.cand_px = static_cast<double2*>(E->cand_px.p), W.keep = static_cast<uint8_t*>(E->keep.p), W.near = static_cast<int32_t*>(E->near.p);
    W.counters = static_cast<int32_t*>(E->counters.p), W.block_count = static_cast<int32_t*>(E->block_count.p);
    W.row_px = static_cast<double2*>(E->row_px.p), W.gidx = static_cast<int32_t*>(E->gidx.p), W.r_lookup = static_cast<int32_t*>(E->r_lookup.p);
    W.nb = static_cast<int32_t*>(E->nb.p);

    const dim3 block(F64_BLOCK);
    hipLaunchKernelGGL(f64_fill_kernel, dim3((M->n_nodes + 1 + F64_BLOCK - 1) / F64_BLOCK), block, 0, s, W.r_lookup, M->n_nodes + 1, -1, W.counters);
    hipLaunchKernelGGL(f64_project_kernel, dim3(n_blocks), block, 0, s, F, W);

    /* the host decides the listed candidates again, and overrules the device where they disagree */
    int32_t counters[4] = {0, 0, 0, 0};
    HIP_TRY64(hipMemcpyAsync(counters, W.counters, sizeof(counters), hipMemcpyDeviceToHost, s));
    HIP_TRY64(hipStreamSynchronize(s));
    const int n_near = counters[1];
    if (n_near > 0) {
        std::vector<int32_t> slots;
        if (n_near <= F64_NEAR_CAP) {
            slots.resize(n_near);
            HIP_TRY64(hipMemcpy(slots.data(), W.near, size_t(n_near) * 4, hipMemcpyDeviceToHost));
        }
        else {  /* more than the list holds: every candidate */
            slots.resize(n_cand);
            for (int p = 0; p < n_cand; ++p) slots[p] = p;
        }
        std::vector<uint8_t> keep(n_cand);
        HIP_TRY64(hipMemcpy(keep.data(), W.keep, n_cand, hipMemcpyDeviceToHost));
        E->listed += int64_t(slots.size());
        bool changed = false;
        for (int32_t p : slots) {
            const int r = int(std::upper_bound(table.begin() + nr, table.begin() + 2 * nr, p) - (table.begin() + nr)) - 1;
            const int node = table[r] + (p - table[size_t(nr) + r]);
            const uint8_t host = uint8_t(vm_host_on_screen_f64(in->Rco, &M->h_rays[size_t(node) * 3], F.projection, F.focal, F.centre, F.ik, F.width, F.height, nullptr));
            if (host != keep[p]) {
                keep[p] = host;
                changed = true;
                ++E->overruled;
            }
        }
        if (changed) HIP_TRY64(hipMemcpy(W.keep, keep.data(), n_cand, hipMemcpyHostToDevice));
    }

    hipLaunchKernelGGL(f64_count_kernel, dim3(n_blocks), block, 0, s, F, W);
    hipLaunchKernelGGL(f64_scan_kernel, dim3(1), block, 0, s, W, n_blocks);
    hipLaunchKernelGGL(f64_scatter_kernel, dim3(n_blocks), block, 0, s, F, W);
    if (M->nn > 0) hipLaunchKernelGGL(f64_neighbourhood_kernel, dim3(unsigned((rows * M->nn + F64_BLOCK - 1) / F64_BLOCK)), block, 0, s, F, W);

    const double* result_rows = nullptr;
    if (classify) {
        double* a = static_cast<double*>(E->feat_a.p);
        double* b = static_cast<double*>(E->feat_b.p);
        hipLaunchKernelGGL(f64_sample_kernel, dim3(unsigned((rows + F64_BLOCK - 1) / F64_BLOCK)), block, 0, s, F, W, a);
        for (const HostLayer64& L : E->layers) {
            launch_layer(L.dev, W.counters, W.nb, M->nn, a, b, int(rows), s);
            std::swap(a, b);
        }
        result_rows = a;
    }
    HIP_TRY64(hipGetLastError());
    HIP_TRY64(hipMemcpyAsync(counters, W.counters, sizeof(counters), hipMemcpyDeviceToHost, s));
    HIP_TRY64(hipStreamSynchronize(s));
    const int V = counters[0];
    out->n_visible = V;
    if (V == 0) return VMHIP_OK;
    if (out->pixel_coordinates) HIP_TRY64(hipMemcpyAsync(out->pixel_coordinates, W.row_px, size_t(V) * 16, hipMemcpyDeviceToHost, s));
    if (out->global_indices) HIP_TRY64(hipMemcpyAsync(out->global_indices, W.gidx, size_t(V) * 4, hipMemcpyDeviceToHost, s));
    if (out->neighbourhood && M->nn > 0) HIP_TRY64(hipMemcpyAsync(out->neighbourhood, W.nb, (size_t(V) + 1) * M->nn * 4, hipMemcpyDeviceToHost, s));
    if (classify && out->classifications)
        HIP_TRY64(hipMemcpyAsync(out->classifications, result_rows, (size_t(V) + 1) * E->n_classes * 8, hipMemcpyDeviceToHost, s));
    HIP_TRY64(hipStreamSynchronize(s));
    return VMHIP_OK;
}

}  // namespace

extern "C" {

int vmhip_engine_create_f64(const vmhip_network_f64* net, int32_t n_neighbours, vmhip_engine_f64** out) {
    if (!out) return fail64(VMHIP_ERR_ARGUMENT, "engine_create_f64: null output");
    *out = nullptr;
    if (n_neighbours < 0 || n_neighbours > 16) return fail64(VMHIP_ERR_ARGUMENT, "engine_create_f64: unsupported neighbour count");
    int n_dev = 0;
    HIP_TRY64(hipGetDeviceCount(&n_dev));
    if (n_dev <= 0) return fail64(VMHIP_ERR_HIP, "engine_create_f64: no HIP device");
    vmhip_engine_f64* E = new vmhip_engine_f64();
    E->nn = n_neighbours;
    auto bail = [&](int code, const std::string& msg) {
        vmhip_engine_destroy_f64(E);
        return fail64(code, msg);
    };
    if (hipStreamCreate(&E->stream) != hipSuccess) return bail(VMHIP_ERR_HIP, "engine_create_f64: no stream");
    int width = 4, li = 0;
    for (int g = 0; net && g < net->n_groups; ++g) {
        if (net->group_sizes[g] <= 0) return bail(VMHIP_ERR_ARGUMENT, "engine_create_f64: empty convolutional group");
        for (int l = 0; l < net->group_sizes[g]; ++l, ++li) {
            const vmhip_layer_f64& L = net->layers[li];
            const int slots = l == 0 ? n_neighbours + 1 : 1;
            if (L.n_in != slots * width || L.n_out <= 0 || !L.weights || !L.biases)
                return bail(VMHIP_ERR_ARGUMENT, "engine_create_f64: layer " + std::to_string(li) + " expects " + std::to_string(slots * width)
                                                  + " inputs, has " + std::to_string(L.n_in));
            if (L.activation < VMHIP_SELU || L.activation > VMHIP_TANH) return bail(VMHIP_ERR_ARGUMENT, "engine_create_f64: unknown activation");
            if (L.activation == VMHIP_SOFTMAX && L.n_out > F64_MAX_SOFTMAX)
                return bail(VMHIP_ERR_ARGUMENT, "engine_create_f64: a softmax layer has at most " + std::to_string(F64_MAX_SOFTMAX) + " outputs");
            HostLayer64 H;
            Layer64& D = H.dev;
            D.c_in = width, D.c_in_pad = (width + 3) / 4 * 4, D.n_out = L.n_out, D.n_pad = (L.n_out + 15) / 16 * 16;
            D.slots = slots, D.activation = L.activation;
            std::vector<double> w(size_t(slots) * D.c_in_pad * D.n_pad, 0.0), b(D.n_pad, 0.0);
            for (int s = 0; s < slots; ++s)
                for (int c = 0; c < width; ++c)
                    std::memcpy(&w[(size_t(s) * D.c_in_pad + c) * D.n_pad], L.weights + (size_t(s) * width + c) * L.n_out, sizeof(double) * L.n_out);
            std::memcpy(b.data(), L.biases, sizeof(double) * L.n_out);
            if (hipMalloc(&H.d_w, w.size() * 8) != hipSuccess || hipMalloc(&H.d_b, b.size() * 8) != hipSuccess) {
                if (H.d_w) (void) hipFree(H.d_w);
                return bail(VMHIP_ERR_HIP, "engine_create_f64: out of device memory");
            }
            D.w = H.d_w, D.b = H.d_b;
            E->layers.push_back(H);
            if (hipMemcpy(H.d_w, w.data(), w.size() * 8, hipMemcpyHostToDevice) != hipSuccess
                || hipMemcpy(H.d_b, b.data(), b.size() * 8, hipMemcpyHostToDevice) != hipSuccess)
                return bail(VMHIP_ERR_HIP, "engine_create_f64: weight upload failed");
            width = L.n_out;
            E->max_width = std::max(E->max_width, width);
        }
    }
    E->n_classes = width;
    *out = E;
    return VMHIP_OK;
}

void vmhip_engine_destroy_f64(vmhip_engine_f64* E) {
    if (!E) return;
    if (E->stream) (void) hipStreamSynchronize(E->stream);
    for (HostLayer64& L : E->layers) {
        if (L.d_w) (void) hipFree(L.d_w);
        if (L.d_b) (void) hipFree(L.d_b);
    }
    for (Buf64* b : {&E->ranges, &E->cand_px, &E->keep, &E->near, &E->counters, &E->block_count, &E->row_px, &E->gidx, &E->r_lookup, &E->nb,
                     &E->feat_a, &E->feat_b, &E->image})
        b->release();
    if (E->stream) (void) hipStreamDestroy(E->stream);
    delete E;
}

int32_t vmhip_engine_n_classes_f64(const vmhip_engine_f64* E) { return E ? E->n_classes : 0; }

int vmhip_mesh_upload_f64(const double* rays, const int32_t* neighbours, int32_t n_nodes, int32_t n_neighbours, vmhip_mesh_f64** out) {
    if (!out) return fail64(VMHIP_ERR_ARGUMENT, "mesh_upload_f64: null output");
    *out = nullptr;
    if (!rays || !neighbours || n_nodes <= 0 || n_neighbours <= 0 || n_neighbours > 16) return fail64(VMHIP_ERR_ARGUMENT, "mesh_upload_f64: bad mesh");
    for (size_t i = 0; i < size_t(n_nodes) * n_neighbours; ++i)
        if (neighbours[i] < 0 || neighbours[i] > n_nodes) return fail64(VMHIP_ERR_ARGUMENT, "mesh_upload_f64: neighbour index outside the mesh");
    vmhip_mesh_f64* M = new vmhip_mesh_f64();
    M->n_nodes = n_nodes, M->nn = n_neighbours;
    M->h_rays.assign(rays, rays + size_t(n_nodes) * 3);
    if (hipMalloc(&M->d_rays, size_t(n_nodes) * 24) != hipSuccess || hipMalloc(&M->d_nbr, size_t(n_nodes) * n_neighbours * 4) != hipSuccess
        || hipMemcpy(M->d_rays, rays, size_t(n_nodes) * 24, hipMemcpyHostToDevice) != hipSuccess
        || hipMemcpy(M->d_nbr, neighbours, size_t(n_nodes) * n_neighbours * 4, hipMemcpyHostToDevice) != hipSuccess) {
        vmhip_mesh_release_f64(M);
        return fail64(VMHIP_ERR_HIP, "mesh_upload_f64: device allocation or copy failed");
    }
    *out = M;
    return VMHIP_OK;
}

void vmhip_mesh_release_f64(vmhip_mesh_f64* M) {
    if (!M) return;
    if (M->d_rays) (void) hipFree(M->d_rays);
    if (M->d_nbr) (void) hipFree(M->d_nbr);
    delete M;
}

int vmhip_project_f64(vmhip_engine_f64* E, const vmhip_frame_f64* frame, vmhip_result_f64* result) { return run64(E, frame, result, false); }
int vmhip_classify_f64(vmhip_engine_f64* E, const vmhip_frame_f64* frame, vmhip_result_f64* result) { return run64(E, frame, result, true); }

int vmhip_engine_guard_stats_f64(const vmhip_engine_f64* E, int64_t* listed, int64_t* overruled) {
    if (!E) return fail64(VMHIP_ERR_ARGUMENT, "guard_stats_f64: null engine");
    if (listed) *listed = E->listed;
    if (overruled) *overruled = E->overruled;
    return VMHIP_OK;
}
}

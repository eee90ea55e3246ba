/*
 * conv.hip - graph-convolution layers for gfx950: neighbour gather + dense + bias + activation fused in
 * one kernel per layer (reference engine/cpu/engine.hpp:213-264, apply_activation.hpp:34-84).
 *
 * Row r of the output is act(b + sum over slots s and channels c of in[src(r, s)][c] * W[s*C_in + c][:])
 * with src(r, 0) = r and src(r, s) = neighbourhood[r][s-1]; the null row (r = V) is an ordinary row whose
 * neighbours all point to itself. The gathered matrix is never materialised.
 *
 * vm_conv_rows_kernel<C_IN, C_OUT, SLOTS>: one row per lane, C_OUT accumulators in registers, the weight
 *   matrix read through wave-uniform addresses (scalar loads, one weight feeds 64 rows per instruction).
 * vm_conv_generic_kernel: any shape, output channels in chunks of 8; the fallback for shapes that have no
 *   specialisation.
 */
#include <atomic>
#include <cstdio>
#include <map>
#include <mutex>
#include <string>

#include "vmhip_internal.h"

namespace {

__device__ __forceinline__ int find_frame_by_row_tile(const VmFrame* frames, int n, int tile) {
    int lo = 0, hi = n - 1;
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (frames[mid].row_tile0 <= tile) lo = mid;
        else hi = mid - 1;
    }
    return lo;
}

__device__ __forceinline__ float selu(float s) {
    const float lambda = 1.0507009873554804934193349852946f;
    const float alpha = 1.6732632423543772848170429916717f;
    return lambda * (s >= 0.0f ? s : alpha * expf(s) - alpha);
}

template <int C_OUT>
__device__ __forceinline__ void activate(float (&acc)[C_OUT], int activation) {
    switch (activation) {
        case VMHIP_SELU:
#pragma unroll
            for (int o = 0; o < C_OUT; ++o) acc[o] = selu(acc[o]);
            break;
        case VMHIP_RELU:
#pragma unroll
            for (int o = 0; o < C_OUT; ++o) acc[o] = fmaxf(acc[o], 0.0f);
            break;
        case VMHIP_TANH:
#pragma unroll
            for (int o = 0; o < C_OUT; ++o) acc[o] = tanhf(acc[o]);
            break;
        default: { /* softmax without max subtraction, as the reference */
            float sum = 0.0f;
#pragma unroll
            for (int o = 0; o < C_OUT; ++o) {
                acc[o] = expf(acc[o]);
                sum += acc[o];
            }
#pragma unroll
            for (int o = 0; o < C_OUT; ++o) acc[o] = acc[o] / sum;
        } break;
    }
}

template <int C_IN, int C_OUT, int SLOTS>
__global__ __launch_bounds__(VMHIP_TILE) void vm_conv_rows_kernel(VmBatchDev B, VmLayerDev L, const float* __restrict__ in,
                                                                  float* __restrict__ out) {
    const int tile = blockIdx.x;
    if (tile >= vm_row_tiles(B)) return; /* the grid may be sized for more tiles than the staged batch has */
    const int f = find_frame_by_row_tile(B.frames, B.n_frames, tile);
    const VmFrame& F = B.frames[f];
    const int V = B.frame_V[f];
    const int i = (tile - F.row_tile0) * VMHIP_TILE + threadIdx.x;
    if (i > V) return;
    const size_t row = (size_t) F.row_base + i;
    const float* __restrict__ w = L.w;

    float acc[C_OUT];
#pragma unroll
    for (int o = 0; o < C_OUT; ++o) acc[o] = L.b[o];

    constexpr int SLOT_UNROLL = C_IN * C_OUT >= 512 ? 1 : SLOTS;
    /* the slot loop stays rolled for the big shapes: fully unrolled they are tens of thousands of FMAs */
#pragma unroll SLOT_UNROLL
    for (int s = 0; s < SLOTS; ++s) {
        const size_t src = s == 0 ? row : (size_t) F.row_base + B.row_nb[row * B.nb_stride + (s - 1)];
        const float* __restrict__ x = in + src * C_IN;
        float v[C_IN];
        if (C_IN % 4 == 0) {
#pragma unroll
            for (int c = 0; c < C_IN; c += 4) {
                const float4 t = *reinterpret_cast<const float4*>(x + c);
                v[c] = t.x, v[c + 1] = t.y, v[c + 2] = t.z, v[c + 3] = t.w;
            }
        }
        else {
#pragma unroll
            for (int c = 0; c < C_IN; ++c) v[c] = x[c];
        }
#pragma unroll
        for (int c = 0; c < C_IN; ++c) {
            const float* __restrict__ wr = w + (size_t) (s * C_IN + c) * C_OUT;
#pragma unroll
            for (int o = 0; o < C_OUT; ++o) acc[o] = fmaf(v[c], wr[o], acc[o]);
        }
    }
    activate<C_OUT>(acc, L.activation);

    float* __restrict__ y = out + row * C_OUT;
    if (C_OUT % 4 == 0) {
#pragma unroll
        for (int o = 0; o < C_OUT; o += 4) *reinterpret_cast<float4*>(y + o) = make_float4(acc[o], acc[o + 1], acc[o + 2], acc[o + 3]);
    }
    else {
#pragma unroll
        for (int o = 0; o < C_OUT; ++o) y[o] = acc[o];
    }
}

/* Any shape. Softmax needs the whole row, so it is finished by a second pass over the row's own output. */
__global__ __launch_bounds__(VMHIP_TILE) void vm_conv_generic_kernel(VmBatchDev B, VmLayerDev L, const float* __restrict__ in,
                                                                     float* __restrict__ out) {
    const int tile = blockIdx.x;
    if (tile >= vm_row_tiles(B)) return; /* the grid may be sized for more tiles than the staged batch has */
    const int f = find_frame_by_row_tile(B.frames, B.n_frames, tile);
    const VmFrame& F = B.frames[f];
    const int V = B.frame_V[f];
    const int i = (tile - F.row_tile0) * VMHIP_TILE + threadIdx.x;
    if (i > V) return;
    const size_t row = (size_t) F.row_base + i;
    const int C_IN = L.c_in, C_OUT = L.c_out;
    float* __restrict__ y = out + row * C_OUT;

    for (int o0 = 0; o0 < C_OUT; o0 += 8) {
        float acc[8];
#pragma unroll
        for (int o = 0; o < 8; ++o) acc[o] = o0 + o < C_OUT ? L.b[o0 + o] : 0.0f;
        for (int s = 0; s < L.slots; ++s) {
            const size_t src = s == 0 ? row : (size_t) F.row_base + B.row_nb[row * B.nb_stride + (s - 1)];
            const float* __restrict__ x = in + src * C_IN;
            for (int c = 0; c < C_IN; ++c) {
                const float v = x[c];
                const float* __restrict__ wr = L.w + (size_t) (s * C_IN + c) * C_OUT + o0;
#pragma unroll
                for (int o = 0; o < 8; ++o)
                    if (o0 + o < C_OUT) acc[o] = fmaf(v, wr[o], acc[o]);
            }
        }
#pragma unroll
        for (int o = 0; o < 8; ++o) {
            if (o0 + o < C_OUT) {
                float a = acc[o];
                switch (L.activation) {
                    case VMHIP_SELU: a = selu(a); break;
                    case VMHIP_RELU: a = fmaxf(a, 0.0f); break;
                    case VMHIP_TANH: a = tanhf(a); break;
                    default: a = expf(a); break;
                }
                y[o0 + o] = a;
            }
        }
    }
    if (L.activation == VMHIP_SOFTMAX) {
        float sum = 0.0f;
        for (int o = 0; o < C_OUT; ++o) sum += y[o];
        for (int o = 0; o < C_OUT; ++o) y[o] = y[o] / sum;
    }
}

template <int C_IN, int C_OUT, int SLOTS>
void launch_rows(const VmBatchDev& B, const VmLayerDev& L, const float* in, float* out, hipStream_t stream) {
    hipLaunchKernelGGL((vm_conv_rows_kernel<C_IN, C_OUT, SLOTS>), dim3(B.n_row_tiles), dim3(VMHIP_TILE), 0, stream, B, L, in,
                       out);
}

}  // namespace

int vm_launch_conv(const VmBatchDev& B, const VmLayerDev& L, const float* in, float* out, hipStream_t stream,
                   const char** kernel_name) {
    if (B.n_row_tiles <= 0) return 0;
#define ROWS_CASE(CI, CO, SL)                                   \
    if (L.c_in == CI && L.c_out == CO && L.slots == SL) {       \
        launch_rows<CI, CO, SL>(B, L, in, out, stream);         \
        if (kernel_name) *kernel_name = "conv_rows_" #CI "x" #CO "s" #SL; \
        return 0;                                               \
    }
    /* Ring6 (7 slots) */
    ROWS_CASE(4, 16, 7)
    ROWS_CASE(16, 16, 7)
    ROWS_CASE(16, 2, 7)
    ROWS_CASE(16, 32, 7)
    ROWS_CASE(32, 32, 7)
    ROWS_CASE(32, 16, 7)
    ROWS_CASE(16, 3, 7)
    ROWS_CASE(4, 64, 7)
    ROWS_CASE(64, 64, 7)
    ROWS_CASE(16, 8, 7)
    ROWS_CASE(8, 8, 7)
    ROWS_CASE(8, 5, 7)
    /* NMGrid8 (9 slots) */
    ROWS_CASE(4, 24, 9)
    ROWS_CASE(24, 24, 9)
    ROWS_CASE(24, 4, 9)
#undef ROWS_CASE
    /* no kernel knows this shape at compile time: one row per lane with loops over run-time widths. Said once per
     * process, so that a network that lands here by accident (an input width that is not a multiple of four channels,
     * more than 64 output channels, a gather of neither 7 nor 9 slots) is noticed. */
    static std::atomic<bool> told{false};
    if (!told.exchange(true))
        fprintf(stderr, "visualmesh_hip: layer %d -> %d (%d gather slots) has no matrix-core kernel; it runs on the generic one-row-per-lane kernel\n",
                L.c_in, L.c_out, L.slots);
    hipLaunchKernelGGL(vm_conv_generic_kernel, dim3(B.n_row_tiles), dim3(VMHIP_TILE), 0, stream, B, L, in, out);
    if (kernel_name) *kernel_name = "conv_generic";
    return 0;
}

const char* vm_kernel_name(const char* family, int c_in, int c_out, int slots) {
    static std::mutex guard;
    static std::map<std::string, std::string> names; /* node addresses of a map stay put */
    char text[96];
    snprintf(text, sizeof(text), "%s_%dx%ds%d", family, c_in, c_out, slots);
    std::lock_guard<std::mutex> lock(guard);
    return names.emplace(text, text).first->second.c_str();
}

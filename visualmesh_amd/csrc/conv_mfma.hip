/*
 * conv_mfma.hip - graph-convolution layers on the matrix cores of gfx950 (v_mfma_f32_16x16x4_f32, fp32 in,
 * fp32 accumulate): neighbour gather + dense + bias + activation in one kernel
 * (reference engine/cpu/engine.hpp:213-264, apply_activation.hpp:34-84).
 *
 * Shape of the contraction: out[row][o] = b[o] + sum_{s, c} in[src(row, s)][c] * W[s*C_IN + c][o].
 * One MFMA computes a 16 (output channels) x 16 (rows) block over 4 values of the reduction index:
 *   A operand: lane l supplies W[k(l / 16)][o = l % 16]
 *   B operand: lane l supplies in[src(row = l % 16)][k(l / 16)]
 *   D:         lane l holds out channels 4 * (l / 16) + {0,1,2,3} of row l % 16   -> one 16-byte store per lane
 * The reduction index is free to be permuted as long as both operands agree, so lane group q = l / 16 takes
 * the q-th quarter of every gathered row: a lane's inputs for one gather slot are C_IN / 4 consecutive floats
 * of one source row, and MFMA step j of slot s uses element j of that run. The weights are stored once, in
 * exactly the order the lanes consume them ([slot][j][column block][lane]), and live in LDS for the life of a
 * block; one LDS read feeds RB MFMAs (RB row blocks per wave).
 *
 * The gathered rows go straight from global memory into registers in operand layout (16-byte loads, no
 * staging). Mesh order is spatially coherent (about 88 % of a row's neighbours lie in the same 256-row tile),
 * so after the XCD-aware tile walk below nearly all of these loads hit in L1/L2 and the HBM traffic is the
 * algorithmic minimum; what the loads still cost is issue slots next to the matrix instructions.
 *
 * Blocks are persistent and XCD aware: hardware deals consecutive workgroups round-robin to the 8 XCDs, each
 * with its own L2. Block b therefore walks a contiguous eighth of the tiles (xcd = b % 8), so the neighbour
 * rows a tile gathers - which lie in nearby tiles, mesh order being spatially coherent - are found in the
 * same L2 instead of being fetched by every XCD.
 */
#include <cstdlib>

#include "vmhip_internal.h"

namespace {

typedef float v4f __attribute__((ext_vector_type(4)));

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

/* loads N consecutive 32-bit words with the widest loads their count allows (the caller guarantees the
 * matching alignment: rows are multiples of 16, 8 or 4 bytes accordingly) */
template <int N>
__device__ __forceinline__ void load_run(const float* __restrict__ p, float (&v)[N]) {
    if constexpr (N % 4 == 0) {
#pragma unroll
        for (int i = 0; i < N; i += 4) {
            const float4 t = *reinterpret_cast<const float4*>(p + i);
            v[i] = t.x, v[i + 1] = t.y, v[i + 2] = t.z, v[i + 3] = t.w;
        }
    }
    else if constexpr (N % 2 == 0) {
#pragma unroll
        for (int i = 0; i < N; i += 2) {
            const float2 t = *reinterpret_cast<const float2*>(p + i);
            v[i] = t.x, v[i + 1] = t.y;
        }
    }
    else {
#pragma unroll
        for (int i = 0; i < N; ++i) v[i] = p[i];
    }
}
template <int N>
__device__ __forceinline__ void load_run(const int32_t* __restrict__ p, int (&v)[N]) {
    if constexpr (N % 4 == 0) {
#pragma unroll
        for (int i = 0; i < N; i += 4) {
            const int4 t = *reinterpret_cast<const int4*>(p + i);
            v[i] = t.x, v[i + 1] = t.y, v[i + 2] = t.z, v[i + 3] = t.w;
        }
    }
    else if constexpr (N % 2 == 0) {
#pragma unroll
        for (int i = 0; i < N; i += 2) {
            const int2 t = *reinterpret_cast<const int2*>(p + i);
            v[i] = t.x, v[i + 1] = t.y;
        }
    }
    else {
#pragma unroll
        for (int i = 0; i < N; ++i) v[i] = p[i];
    }
}

/* Gather-from-global variant. NW waves per block, RB row blocks of 16 rows per wave: NW * RB * 16 == VMHIP_TILE.
 *
 * Each wave walks its tiles with a software pipeline, because the per-tile chain "which frame -> how many rows
 * -> neighbour table -> source rows" is four dependent memory round trips and the waves that share a SIMD tend
 * to run in lockstep (the matrix pipe is served round-robin), so a chain left in the open idles the pipe for
 * every wave at once:
 *   - the frame lookup and the neighbour-table loads of tile t+1 are issued before the matrix work of tile t;
 *   - the slot-0 rows of tile t+1 are requested during the last slot of tile t, ahead of tile t's epilogue;
 *   - inside a tile, slot s+1's rows are requested before slot s's matrix instructions (fenced so the
 *     scheduler cannot sink the loads back next to their uses). */
template <int C_IN, int C_OUT, int SLOTS, int NW, int RB>
__global__ __launch_bounds__(NW * 64) void vm_conv_mfma_kernel(VmBatchDev B, VmLayerDev L, const float* __restrict__ in,
                                                               float* __restrict__ out) {
    static_assert(C_IN % 4 == 0, "a lane group takes a quarter of each gathered row");
    static_assert(NW * RB * 16 == VMHIP_TILE, "a block covers one tile");
    constexpr int KQ = C_IN / 4;              /* floats per lane per slot */
    constexpr int CB = (C_OUT + 15) / 16;     /* column blocks of 16 output channels */
    constexpr int NN = SLOTS - 1;
    constexpr int NBV = NN > 0 ? NN : 1;
    constexpr int W_FLOATS = SLOTS * KQ * CB * 64;

    extern __shared__ float w_lds[];
    for (int i = threadIdx.x * 4; i < W_FLOATS; i += NW * 64 * 4)
        *reinterpret_cast<float4*>(w_lds + i) = *reinterpret_cast<const float4*>(L.w_mfma + i);
    __syncthreads();

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int q = lane >> 4;   /* quarter of the gathered row / group of 4 output channels */
    const int r16 = lane & 15; /* row within a row block / output channel within a column block */
    const int activation = L.activation;

    v4f bias[CB];
#pragma unroll
    for (int cb = 0; cb < CB; ++cb) {
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int o = cb * 16 + q * 4 + v;
            bias[cb][v] = o < C_OUT ? L.b[o] : 0.0f;
        }
    }

    /* persistent, XCD-aware walk over the tiles */
    const int n_tiles = B.n_row_tiles;
    const int xcd = blockIdx.x & 7, lb = blockIdx.x >> 3, gx = gridDim.x >> 3;
    const int per_xcd = (n_tiles + 7) >> 3;
    const int t_end = min(n_tiles, (xcd + 1) * per_xcd);

    /* wave-uniform description of a tile: the frame's first row, its visible count, the wave's first row */
    struct Info {
        uint32_t base;
        int V;
        int row0;
    };
    auto describe = [&](int tile) {
        const int f = find_frame_by_row_tile(B.frames, B.n_frames, tile);
        const VmFrame& F = B.frames[f];
        Info t;
        t.base = (uint32_t) F.row_base;
        t.V = B.frame_V[f];
        t.row0 = (tile - F.row_tile0) * VMHIP_TILE + wave * (RB * 16);
        return t;
    };
    /* the lane's rows of a tile, clamped to the null row (lanes past it compute on its data and skip the store) */
    auto request_neighbours = [&](const Info& t, int (&nb)[RB][NBV]) {
        if constexpr (NN > 0) {
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) {
                const uint32_t row = t.base + (uint32_t) max(0, min(t.row0 + rb * 16 + r16, t.V));
                load_run<NN>(B.row_nb + (size_t) row * B.nb_stride, nb[rb]);
            }
        }
    };
    auto resolve = [&](const Info& t, const int (&nb)[RB][NBV], uint32_t (&src)[RB][SLOTS], bool (&valid)[RB]) {
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
            const int i = t.row0 + rb * 16 + r16;
            valid[rb] = i <= t.V;
            src[rb][0] = t.base + (uint32_t) max(0, min(i, t.V));
#pragma unroll
            for (int s = 0; s < NN; ++s) src[rb][s + 1] = t.base + (uint32_t) nb[rb][s];
        }
    };

    int tile = xcd * per_xcd + lb;
    if (tile >= t_end) return;

    Info cur = describe(tile);
    int nb[RB][NBV];
    request_neighbours(cur, nb);
    uint32_t src[RB][SLOTS];
    bool valid[RB];
    resolve(cur, nb, src, valid);
    float x[2][RB][KQ];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) load_run<KQ>(in + (size_t) src[rb][0] * C_IN + q * KQ, x[0][rb]);

    int next = tile + gx;
    Info nxt = cur;
    if (next < t_end) {
        nxt = describe(next);
        request_neighbours(nxt, nb);
    }

    while (true) {
        const bool has_next = next < t_end;
        uint32_t src_next[RB][SLOTS];
        bool valid_next[RB];

        v4f acc[RB][CB];
#pragma unroll
        for (int rb = 0; rb < RB; ++rb)
#pragma unroll
            for (int cb = 0; cb < CB; ++cb) acc[rb][cb] = bias[cb];

#pragma unroll
        for (int s = 0; s < SLOTS; ++s) {
            const int cur_buf = s & 1;
            if (s + 1 < SLOTS) {
#pragma unroll
                for (int rb = 0; rb < RB; ++rb) load_run<KQ>(in + (size_t) src[rb][s + 1] * C_IN + q * KQ, x[cur_buf ^ 1][rb]);
            }
            else if (has_next) {
                /* last slot: the other buffer is free; fill it with the next tile's slot 0 */
                resolve(nxt, nb, src_next, valid_next);
#pragma unroll
                for (int rb = 0; rb < RB; ++rb) load_run<KQ>(in + (size_t) src_next[rb][0] * C_IN + q * KQ, x[cur_buf ^ 1][rb]);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int j = 0; j < KQ; ++j) {
#pragma unroll
                for (int cb = 0; cb < CB; ++cb) {
                    const float a = w_lds[((s * KQ + j) * CB + cb) * 64 + lane];
#pragma unroll
                    for (int rb = 0; rb < RB; ++rb)
                        acc[rb][cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, x[cur_buf][rb][j], acc[rb][cb], 0, 0, 0);
                }
            }
        }

        /* look one more tile ahead before the epilogue: frame lookup + neighbour table of tile t+2 */
        const int after = next + gx;
        Info nxt2 = nxt;
        if (has_next && after < t_end) {
            nxt2 = describe(after);
            request_neighbours(nxt2, nb);
        }
        __builtin_amdgcn_sched_barrier(0);

        /* activation and store: lane holds channels cb*16 + q*4 + {0..3} of row rb*16 + r16 */
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
            if (activation == VMHIP_SOFTMAX) {
                float sum = 0.0f;
#pragma unroll
                for (int cb = 0; cb < CB; ++cb)
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        const bool real = cb * 16 + q * 4 + v < C_OUT;
                        const float e = real ? expf(acc[rb][cb][v]) : 0.0f;
                        acc[rb][cb][v] = e;
                        sum += e;
                    }
                sum += __shfl_xor(sum, 16);
                sum += __shfl_xor(sum, 32);
#pragma unroll
                for (int cb = 0; cb < CB; ++cb)
#pragma unroll
                    for (int v = 0; v < 4; ++v) acc[rb][cb][v] = acc[rb][cb][v] / sum;
            }
            else {
#pragma unroll
                for (int cb = 0; cb < CB; ++cb)
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        const float a = acc[rb][cb][v];
                        acc[rb][cb][v] = activation == VMHIP_SELU ? selu(a) : activation == VMHIP_RELU ? fmaxf(a, 0.0f) : tanhf(a);
                    }
            }
            if (valid[rb]) {
                float* __restrict__ y = out + (size_t) src[rb][0] * C_OUT; /* valid => src[rb][0] is the lane's own row */
#pragma unroll
                for (int cb = 0; cb < CB; ++cb) {
                    const int o = cb * 16 + q * 4;
                    if (C_OUT % 4 == 0) {
                        if (o < C_OUT) *reinterpret_cast<float4*>(y + o) = make_float4(acc[rb][cb][0], acc[rb][cb][1], acc[rb][cb][2], acc[rb][cb][3]);
                    }
                    else {
#pragma unroll
                        for (int v = 0; v < 4; ++v)
                            if (o + v < C_OUT) y[o + v] = acc[rb][cb][v];
                    }
                }
            }
        }

        if (!has_next) break;
        /* rotate: the next tile becomes current; its slot 0 sits in the buffer the last slot left free */
        constexpr int LAST = (SLOTS - 1) & 1;
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
            valid[rb] = valid_next[rb];
#pragma unroll
            for (int s = 0; s < SLOTS; ++s) src[rb][s] = src_next[rb][s];
            if (LAST == 0) {
#pragma unroll
                for (int j = 0; j < KQ; ++j) x[0][rb][j] = x[1][rb][j];
            }
        }
        tile = next;
        next = after;
        nxt = nxt2;
    }
}


template <int C_IN, int C_OUT, int SLOTS, int NW, int RB>
int launch_mfma(const VmBatchDev& B, const VmLayerDev& L, const float* in, float* out, hipStream_t stream) {
    constexpr int KQ = C_IN / 4, CB = (C_OUT + 15) / 16;
    constexpr size_t lds = size_t(SLOTS) * KQ * CB * 64 * sizeof(float);
    auto kernel = vm_conv_mfma_kernel<C_IN, C_OUT, SLOTS, NW, RB>;
    static bool configured = false;
    if (!configured) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, int(lds)) != hipSuccess) {
            (void) hipGetLastError();
            return -1;
        }
        configured = true;
    }
    /* blocks per CU limited by LDS (160 KB per CU) and registers; 8 XCDs x 32 CUs */
    int per_cu = int((160 * 1024) / (lds + 512));
    per_cu = per_cu < 1 ? 1 : per_cu > (NW == 4 ? 3 : 2) ? (NW == 4 ? 3 : 2) : per_cu;
    if (const char* e = getenv("VMHIP_MFMA_BLOCKS_PER_CU")) per_cu = atoi(e) > 0 ? atoi(e) : per_cu;
    int grid = 256 * per_cu;
    const int need = ((B.n_row_tiles + 7) / 8) * 8;
    if (grid > need) grid = need;
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(NW * 64), lds, stream, B, L, in, out);
    return 0;
}

template <int C_IN, int C_OUT, int SLOTS>
int launch_pick(const VmBatchDev& B, const VmLayerDev& L, const float* in, float* out, hipStream_t stream) {
    /* 8 waves x 2 row blocks: 16 accumulator registers and two 16-register input buffers per lane leave room
     * for four waves per SIMD on the 32-wide layers */
    return launch_mfma<C_IN, C_OUT, SLOTS, 8, 2>(B, L, in, out, stream);
}

}  // namespace

/* Permuted weight layout the kernel consumes: [slot][j][column block][lane = q*16 + o] with
 * value W[slot*C_IN + q*(C_IN/4) + j][cb*16 + o], zero for padded output channels. */
size_t vm_mfma_weight_floats(int c_in, int c_out, int slots) { return size_t(slots) * (c_in / 4) * ((c_out + 15) / 16) * 64; }
void vm_mfma_permute_weights(const float* w, int c_in, int c_out, int slots, float* wp) {
    const int KQ = c_in / 4, CB = (c_out + 15) / 16;
    for (int s = 0; s < slots; ++s)
        for (int j = 0; j < KQ; ++j)
            for (int cb = 0; cb < CB; ++cb)
                for (int q = 0; q < 4; ++q)
                    for (int o = 0; o < 16; ++o) {
                        const int col = cb * 16 + o;
                        const int k = s * c_in + q * KQ + j;
                        wp[((size_t(s) * KQ + j) * CB + cb) * 64 + q * 16 + o] = col < c_out ? w[size_t(k) * c_out + col] : 0.0f;
                    }
}

bool vm_mfma_supported(int c_in, int c_out, int slots) {
#define MFMA_SHAPE(CI, CO, SL) \
    if (c_in == CI && c_out == CO && slots == SL) return true;
#include "conv_mfma_shapes.inc"
#undef MFMA_SHAPE
    return false;
}

int vm_launch_conv_mfma(const VmBatchDev& B, const VmLayerDev& L, const float* in, float* out, hipStream_t stream,
                        const char** kernel_name) {
    if (B.n_row_tiles <= 0) return 0;
#define MFMA_SHAPE(CI, CO, SL)                                                                 \
    if (L.c_in == CI && L.c_out == CO && L.slots == SL) {                                      \
        if (kernel_name) *kernel_name = "conv_mfma_" #CI "x" #CO "s" #SL;                      \
        return launch_pick<CI, CO, SL>(B, L, in, out, stream);                                 \
    }
#include "conv_mfma_shapes.inc"
#undef MFMA_SHAPE
    return -1;
}

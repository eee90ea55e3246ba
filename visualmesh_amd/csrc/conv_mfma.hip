/*
 * conv_mfma.hip - graph-convolution layers on the matrix cores of gfx950: neighbour gather + dense + bias +
 * activation in one kernel (reference engine/cpu/engine.hpp:213-264, apply_activation.hpp:34-84).
 *
 * Shape of the contraction: out[row][o] = b[o] + sum_{s, c} in[src(row, s)][c] * W[s*C_IN + c][o].
 * One MFMA computes a 16 (output channels) x 16 (rows) block over a few values of the reduction index:
 *   A operand: lane l supplies W[k(l / 16)][o = l % 16]
 *   B operand: lane l supplies in[src(row = l % 16)][k(l / 16)]
 *   D:         lane l holds out channels 4 * (l / 16) + {0,1,2,3} of row l % 16   -> one vector store per lane
 * The instruction is v_mfma_f32_16x16x4_f32: one float per lane and step, 4 reduction values per instruction (the bf16
 * engine's layers have a kernel of their own, conv_bf16.hip).
 * The reduction index is free to be permuted as long as both operands agree, so lane group q = l / 16 takes
 * the q-th quarter of every gathered row: a lane's inputs for one gather slot are C_IN / 4 consecutive values
 * of one source row, and step j of slot s uses the j-th register of that run. The weights are stored once, in
 * exactly the order the lanes consume them ([slot][step][column block][lane]), and live in LDS for the life of
 * a block; one LDS read feeds RB MFMAs (RB row blocks per wave).
 *
 * The gathered rows go straight from global memory into registers in operand layout (16-byte loads, no
 * staging). Mesh order is spatially coherent (about 88 % of a row's neighbours lie in the same 256-row tile),
 * so with the XCD-aware tile walk nearly all of these loads hit in L1/L2 and the HBM traffic is the algorithmic
 * minimum; what the loads still cost is issue slots next to the matrix instructions.
 *
 * Blocks are persistent and XCD aware: hardware deals consecutive workgroups round-robin to the 8 XCDs, each
 * with its own L2. Block b therefore walks a contiguous eighth of the tiles (xcd = b % 8), so the neighbour
 * rows a tile gathers are found in the same L2 instead of being fetched by every XCD.
 *
 * Each wave walks its tiles with a software pipeline, because the per-tile chain "which frame -> how many rows
 * -> neighbour table -> source rows" is four dependent memory round trips:
 *   - the frame lookup and the neighbour-table loads of tile t+2 are issued before the epilogue of tile t;
 *   - the slot-0 rows of tile t+1 are requested during the last slot of tile t;
 *   - inside a tile, slot s+1's rows are requested before slot s's matrix instructions (fenced so the
 *     scheduler cannot sink the loads back next to their uses).
 */
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <type_traits>

#include <atomic>

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

/* selu with the hardware exponential (v_exp_f32 on s * log2 e): the branch that needs it has s < 0, where the
 * result alpha * e^s - alpha is off by at most ~3e-7 absolute against the correctly rounded one, two orders of
 * magnitude inside the 1e-4 gate on the probabilities, and it takes 6 instructions per value instead of ~20 (the
 * activation is a visible share of a layer's time: a wave's vector instructions do not overlap its own matrix
 * instructions). */
__device__ __forceinline__ float selu(float s) {
    const float lambda = 1.0507009873554804934193349852946f;
    const float alpha = 1.6732632423543772848170429916717f;
    return lambda * (s >= 0.0f ? s : alpha * __builtin_amdgcn_exp2f(s * 1.44269504088896340736f) - alpha);
}

/* N consecutive 32-bit words with the widest loads their count allows (the caller guarantees the matching
 * alignment: runs start at multiples of 16, 8 or 4 bytes accordingly) */
template <typename T, int N>
__device__ __forceinline__ void load_words(const T* __restrict__ p, T (&v)[N]) {
    static_assert(sizeof(T) == 4, "32-bit words");
    if constexpr (N % 4 == 0) {
        typedef T vec4 __attribute__((ext_vector_type(4)));
#pragma unroll
        for (int i = 0; i < N; i += 4) {
            const vec4 t = *reinterpret_cast<const vec4*>(p + i);
            v[i] = t.x, v[i + 1] = t.y, v[i + 2] = t.z, v[i + 3] = t.w;
        }
    }
    else if constexpr (N % 2 == 0) {
        typedef T vec2 __attribute__((ext_vector_type(2)));
#pragma unroll
        for (int i = 0; i < N; i += 2) {
            const vec2 t = *reinterpret_cast<const vec2*>(p + i);
            v[i] = t.x, v[i + 1] = t.y;
        }
    }
    else {
#pragma unroll
        for (int i = 0; i < N; ++i) v[i] = p[i];
    }
}

/* ---- operand policies: how a lane fetches its quarter of a gathered row (load: raw registers, no dependent
 * arithmetic, so that the request can be issued a slot ahead), how the raw registers become matrix operands
 * (prepare: runs when the slot is consumed) and what one reduction step issues (accumulate) ---- */

/* fp32 arithmetic on fp32 rows */
template <int C_IN>
struct OperandF32 {
    static constexpr int STEPS = C_IN / 4;
    static constexpr int PARTS = 1;
    static constexpr int RAW = STEPS;
    typedef float areg_t;
    typedef float raw_t;
    typedef float op_t;
    static __device__ __forceinline__ void load(const void* __restrict__ in, uint32_t row, int q, raw_t (&x)[RAW]) {
        load_words<float, RAW>(reinterpret_cast<const float*>(in) + (size_t) row * C_IN + q * RAW, x);
    }
    static __device__ __forceinline__ void prepare(const raw_t (&x)[RAW], op_t (&b)[STEPS]) {
#pragma unroll
        for (int j = 0; j < STEPS; ++j) b[j] = x[j];
    }
    static __device__ __forceinline__ v4f accumulate(int, areg_t a, op_t b, v4f c) { return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0); }
};

/* four consecutive output channels of one row; C_OUT_T > 0: the row's width is known to the compiler */
template <typename OUT_T, int C_OUT_T>
__device__ __forceinline__ void store4(void* __restrict__ out, uint32_t row, int o, v4f v, int c_out) {
    static_assert(sizeof(OUT_T) == 4, "rows are stored as fp32");
    float* y = reinterpret_cast<float*>(out) + (size_t) row * c_out + o;
    if ((C_OUT_T > 0 ? C_OUT_T : c_out) % 4 == 0) {
        if (o < c_out) *reinterpret_cast<float4*>(y) = make_float4(v[0], v[1], v[2], v[3]);
    }
    else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if (o + i < c_out) y[i] = v[i];
    }
}

/* NW waves per block, RB row blocks of 16 rows per wave: NW * RB * 16 == VMHIP_TILE. */
/* C_OUT_T > 0: that many output channels, known to the compiler. C_OUT_T < 0: -C_OUT_T column blocks of 16 and the
 * layer's own count of output channels (L.c_out) read at run time. */
template <class OP, int C_OUT_T, int SLOTS, typename OUT_T, int NW, int RB>
__global__ __launch_bounds__(NW * 64) void vm_conv_mfma_kernel(VmBatchDev B, VmLayerDev L, const void* __restrict__ in, void* __restrict__ out) {
    static_assert(NW * RB * 16 == VMHIP_TILE, "a block covers one tile");
    constexpr int STEPS = OP::STEPS;
    constexpr int CB = C_OUT_T > 0 ? (C_OUT_T + 15) / 16 : -C_OUT_T; /* column blocks of 16 output channels */
    const int C_OUT = C_OUT_T > 0 ? C_OUT_T : L.c_out;
    constexpr int NN = SLOTS - 1;
    constexpr int NBV = NN > 0 ? NN : 1;
    constexpr int PARTS = OP::PARTS;
    constexpr int W_BYTES = SLOTS * STEPS * CB * PARTS * 64 * (int) sizeof(typename OP::areg_t);
    constexpr int RAW = OP::RAW;
    typedef typename OP::areg_t areg_t;
    typedef typename OP::raw_t raw_t;
    typedef typename OP::op_t op_t;

    extern __shared__ float4 w_lds4[];
    /* G consecutive steps of a lane's weights lie next to each other in LDS, so that one read brings G of them */
    constexpr int G = (PARTS == 1 && sizeof(areg_t) == 4) ? (STEPS % 4 == 0 ? 4 : STEPS % 2 == 0 ? 2 : 1) : 1;
    if constexpr (G == 1) {
        for (int i = threadIdx.x; i < W_BYTES / 16; i += NW * 64) w_lds4[i] = reinterpret_cast<const float4*>(L.w_mfma)[i];
    }
    else {
        float* const w = reinterpret_cast<float*>(w_lds4);
        for (int i = threadIdx.x; i < W_BYTES / 4; i += NW * 64) {
            const int e = i % G, l = (i / G) % 64, cb = (i / (G * 64)) % CB, jg = (i / (G * 64 * CB)) % (STEPS / G), sl = i / (STEPS * 64 * CB);
            w[i] = reinterpret_cast<const float*>(L.w_mfma)[((sl * STEPS + jg * G + e) * CB + cb) * 64 + l];
        }
    }
    __syncthreads();
    const areg_t* w_lds = reinterpret_cast<const areg_t*>(w_lds4);

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
    const int n_tiles = vm_row_tiles(B);
    const int xcd = blockIdx.x & 7, lb = blockIdx.x >> 3, gx = gridDim.x >> 3;
    const int per_xcd = (n_tiles + 7) >> 3;
    const int t_end = min(n_tiles, (xcd + 1) * per_xcd);

    /* wave-uniform description of a tile: the frame's first row, its visible count, the wave's first row */
    struct Info {
        uint32_t base;
        int V;
        int row0;
    };
    /* With the tile descriptors at hand (built next to the neighbourhood table) a tile is described by one 16-byte
     * buffer load: vector memory on purpose, because a scalar load in flight shares its counter with the LDS
     * reads of the weights and would turn each of their waits into a wait for global memory. The values stay in
     * vector registers (all lanes equal). Without descriptors: frame search and visible count by scalar loads. */
    const bool have_desc = B.tile_desc != nullptr;
    const __amdgpu_buffer_rsrc_t desc_rsrc =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<int4*>(B.tile_desc), 0, have_desc ? n_tiles * 16 : 0, 0x00020000);
    auto describe = [&](int tile) {
        Info t;
        if (have_desc) {
            typedef uint32_t v4u __attribute__((ext_vector_type(4)));
            const v4u d = __builtin_amdgcn_raw_buffer_load_b128(desc_rsrc, tile * 16, 0, 0); /* {first row, rows in use, -, frame's first row} */
            const int tile_row0 = (int) d.x - (int) d.w;
            t.base = d.w;
            t.V = tile_row0 + (int) d.y - 1; /* the last row in use: equals V in the frame's last tile, never clamps elsewhere */
            t.row0 = tile_row0 + wave * (RB * 16);
        }
        else {
            const int f = find_frame_by_row_tile(B.frames, B.n_frames, tile);
            const VmFrame& F = B.frames[f];
            t.base = (uint32_t) F.row_base;
            t.V = B.frame_V[f];
            t.row0 = (tile - F.row_tile0) * VMHIP_TILE + wave * (RB * 16);
        }
        return t;
    };
    /* the lane's rows of a tile, clamped to the null row (lanes past it compute on its data and skip the store) */
    auto request_neighbours = [&](const Info& t, int (&nb)[RB][NBV]) {
        if constexpr (NN > 0) {
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) {
                const uint32_t row = t.base + (uint32_t) max(0, min(t.row0 + rb * 16 + r16, t.V));
                load_words<int, NN>(B.row_nb + (size_t) row * B.nb_stride, nb[rb]);
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
    raw_t x[2][RB][RAW];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) OP::load(in, src[rb][0], q, x[0][rb]);

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
                for (int rb = 0; rb < RB; ++rb) OP::load(in, src[rb][s + 1], q, x[cur_buf ^ 1][rb]);
            }
            else if (has_next) {
                /* last slot: the other buffer is free; fill it with the next tile's slot 0 */
                resolve(nxt, nb, src_next, valid_next);
#pragma unroll
                for (int rb = 0; rb < RB; ++rb) OP::load(in, src_next[rb][0], q, x[cur_buf ^ 1][rb]);
            }
            __builtin_amdgcn_sched_barrier(0);
            op_t b[RB][STEPS];
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) OP::prepare(x[cur_buf][rb], b[rb]);
            if constexpr (G == 1) {
#pragma unroll
                for (int j = 0; j < STEPS; ++j) {
#pragma unroll
                    for (int cb = 0; cb < CB; ++cb) {
#pragma unroll
                        for (int part = 0; part < PARTS; ++part) {
                            const areg_t a = w_lds[(((s * STEPS + j) * CB + cb) * PARTS + part) * 64 + lane];
#pragma unroll
                            for (int rb = 0; rb < RB; ++rb) acc[rb][cb] = OP::accumulate(part, a, b[rb][j], acc[rb][cb]);
                        }
                    }
                }
            }
            else {
#pragma unroll
                for (int jg = 0; jg < STEPS / G; ++jg) {
#pragma unroll
                    for (int cb = 0; cb < CB; ++cb) {
                        float a[G];
                        load_words<float, G>(reinterpret_cast<const float*>(w_lds) + ((((s * (STEPS / G) + jg) * CB + cb) * 64 + lane) * G), a);
#pragma unroll
                        for (int e = 0; e < G; ++e)
#pragma unroll
                            for (int rb = 0; rb < RB; ++rb) acc[rb][cb] = OP::accumulate(0, a[e], b[rb][jg * G + e], acc[rb][cb]);
                    }
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
            if (valid[rb]) { /* valid => src[rb][0] is the lane's own row */
#pragma unroll
                for (int cb = 0; cb < CB; ++cb) store4<OUT_T, C_OUT_T>(out, src[rb][0], cb * 16 + q * 4, acc[rb][cb], C_OUT);
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
                for (int j = 0; j < RAW; ++j) x[0][rb][j] = x[1][rb][j];
            }
        }
        tile = next;
        next = after;
        nxt = nxt2;
    }
}

template <class OP, int C_OUT, int SLOTS, typename OUT_T>
int launch_mfma(const VmBatchDev& B, const VmLayerDev& L, const void* in, void* out, hipStream_t stream) {
    constexpr int CB = C_OUT > 0 ? (C_OUT + 15) / 16 : -C_OUT;
    constexpr size_t lds = size_t(SLOTS) * OP::STEPS * CB * OP::PARTS * 64 * sizeof(typename OP::areg_t);
    /* 8 waves x 2 row blocks: 16 accumulator registers per pair of column blocks and two input buffers per
     * lane leave room for four waves per SIMD on the 32-wide layers, two blocks per CU. */
    constexpr int NW = 8, RB = VMHIP_TILE / (16 * NW);
    auto kernel = vm_conv_mfma_kernel<OP, C_OUT, SLOTS, OUT_T, NW, RB>;
    static std::atomic<bool> configured{false}; /* engines on several host threads may get here together */
    if (!configured) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, int(lds)) != hipSuccess) {
            (void) hipGetLastError();
            return -1;
        }
        configured = true;
    }
    /* resident blocks per CU: limited by LDS (160 KB per CU) and by four waves per SIMD; 8 XCDs x 32 CUs */
    int per_cu = int((160 * 1024) / (lds + 512));
    per_cu = per_cu < 1 ? 1 : per_cu > 2 ? 2 : per_cu;
    if (const char* e = getenv("VMHIP_MFMA_BLOCKS_PER_CU")) per_cu = atoi(e) > 0 ? atoi(e) : per_cu;
    int grid = 256 * per_cu;
    const int need = ((B.n_row_tiles + 7) / 8) * 8;
    if (grid > need) grid = need;
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(NW * 64), lds, stream, B, L, in, out);
    return 0;
}

template <int CI, int CO, int SL>
int launch_variant(const VmBatchDev& B, const VmLayerDev& L, const void* in, void* out, hipStream_t stream) {
    return launch_mfma<OperandF32<CI>, CO, SL, float>(B, L, in, out, stream);
}

}  // namespace

/* Weight layout the kernel consumes: [slot][step][column block][lane = q*16 + o], one float per lane:
 * W[slot*C_IN + q*(C_IN/4) + step][cb*16 + o], zeros for padded output channels. */
size_t vm_mfma_weight_bytes(int c_in, int c_out, int slots) {
    const size_t cb = (c_out + 15) / 16;
    return size_t(slots) * (c_in / 4) * cb * 64 * 4;
}
void vm_mfma_permute_weights(const float* w, int c_in, int c_out, int slots, void* wp) {
    const int CB = (c_out + 15) / 16;
    const int quarter = c_in / 4;
    float* dst = reinterpret_cast<float*>(wp);
    for (int s = 0; s < slots; ++s)
        for (int j = 0; j < quarter; ++j)
            for (int cb = 0; cb < CB; ++cb)
                for (int q = 0; q < 4; ++q)
                    for (int o = 0; o < 16; ++o) {
                        const int col = cb * 16 + o;
                        const int k = s * c_in + q * quarter + j;
                        dst[((size_t(s) * quarter + j) * CB + cb) * 64 + q * 16 + o] = col < c_out ? w[size_t(k) * c_out + col] : 0.0f;
                    }
}

/* Instantiated shapes: (C_in, C_out, gather slots). */
#define VM_FOR_EACH_MFMA_VARIANT(X) \
    X(4, 16, 7)                     \
    X(16, 16, 7)                    \
    X(16, 32, 7)                    \
    X(32, 32, 7)                    \
    X(32, 16, 7)                    \
    X(4, 64, 7)                     \
    X(64, 64, 7)                    \
    X(4, 24, 9)                     \
    X(24, 24, 9)

/* Every other shape with input rows of 36 to 64 channels (whole 16-byte pieces) and up to 64 output channels:
 * instantiations that know the input width and the number of 16-channel column blocks and read the exact number of
 * output channels at run time; narrower input rows are conv_lds.hip's. X(C_in, column blocks, slots). */
#define VM_MFMA_ANY_WIDTHS(X, CI) X(CI, 1, 7) X(CI, 2, 7) X(CI, 3, 7) X(CI, 4, 7) X(CI, 1, 9) X(CI, 2, 9) X(CI, 3, 9) X(CI, 4, 9) X(CI, 1, 5) X(CI, 2, 5) X(CI, 3, 5) X(CI, 4, 5)
#define VM_FOR_EACH_MFMA_ANY_SHAPE(X) \
    VM_MFMA_ANY_WIDTHS(X, 36)         \
    VM_MFMA_ANY_WIDTHS(X, 40)         \
    VM_MFMA_ANY_WIDTHS(X, 44)         \
    VM_MFMA_ANY_WIDTHS(X, 48)         \
    VM_MFMA_ANY_WIDTHS(X, 52)         \
    VM_MFMA_ANY_WIDTHS(X, 56)         \
    VM_MFMA_ANY_WIDTHS(X, 60)         \
    VM_MFMA_ANY_WIDTHS(X, 64)

bool vm_mfma_supported(int c_in, int c_out, int slots) {
#define X(CI, CO, SL) \
    if (c_in == CI && c_out == CO && slots == SL) return true;
    VM_FOR_EACH_MFMA_VARIANT(X)
#undef X
    return c_in % 4 == 0 && c_in >= 36 && c_in <= 64 && c_out >= 1 && c_out <= 64 && (slots == 5 || slots == 7 || slots == 9);
}

int vm_launch_conv_mfma(const VmBatchDev& B, const VmLayerDev& L, const void* in, void* out, hipStream_t stream, const char** kernel_name) {
    if (B.n_row_tiles <= 0) return 0;
    if (L.in_bf16 || L.out_bf16 || L.arith_bf16) return -1;
#define X(CI, CO, SL)                                                     \
    if (L.c_in == CI && L.c_out == CO && L.slots == SL) {                 \
        if (kernel_name) *kernel_name = "conv_mfma_" #CI "x" #CO "s" #SL; \
        return launch_variant<CI, CO, SL>(B, L, in, out, stream);         \
    }
    VM_FOR_EACH_MFMA_VARIANT(X)
#undef X
    const int blocks = (L.c_out + 15) / 16;
#define X(CI, CBL, SL)                                                                        \
    if (L.c_in == CI && blocks == CBL && L.slots == SL) {                                     \
        if (kernel_name) *kernel_name = vm_kernel_name("conv_mfma", L.c_in, L.c_out, L.slots); \
        return launch_variant<CI, -CBL, SL>(B, L, in, out, stream);                           \
    }
    VM_FOR_EACH_MFMA_ANY_SHAPE(X)
#undef X
    return -1;
}

/*
 * conv_dma.hip - the LDS-gather graph-convolution kernel with its rows brought into LDS by the memory pipeline
 * itself (buffer_load ... lds, 16 bytes per lane, a gfx950 instruction): neighbour gather + dense + bias +
 * activation in one kernel (reference engine/cpu/engine.hpp:213-264, apply_activation.hpp:34-84).
 *
 * Contraction, operand layout, tile-local tables, XCD-aware persistent tile walk and the side path for neighbours
 * that are not staged are those of conv_lds.hip. What differs is the staging:
 *   - a tile's 256 rows and its halo rows travel from global memory straight into LDS; each lane names the 16
 *     bytes it wants (any address, out of range = zeros) and the wave's 64 pieces land contiguously, so the
 *     XOR swizzle of 128-byte rows and the padding of odd widths are a matter of which piece a lane asks for.
 *     No staging registers, no LDS write phase;
 *   - two row buffers alternate. While tile t is contracted out of one, tile t+1 is already landing in the other,
 *     and after the barrier that ends t's matrix work the loads of tile t+2 are issued into the buffer t used;
 *   - one barrier per tile, placed right after the matrix loop; the activation and the stores of tile t come
 *     after it. At that barrier a wave must have all its own LDS loads complete (s_waitcnt vmcnt(0)); everything
 *     it has in flight then was issued before the matrix loop, so the wait is short, and the stores of tile t are
 *     issued after it and are never waited for.
 * A wave never ends with LDS loads in flight (the LDS could already belong to another block).
 */
#include <cstdlib>
#include <type_traits>

#include <atomic>

#include "vmhip_internal.h"

namespace {

typedef float v4f __attribute__((ext_vector_type(4)));
typedef uint32_t v4u __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) void lds_void;

/* selu with the hardware exponential: the branch that needs it has s < 0, where alpha * e^s - alpha is off by at most
 * ~3e-7 absolute against the correctly rounded result */
__device__ __forceinline__ float selu(float s) {
    const float lambda = 1.0507009873554804934193349852946f;
    const float alpha = 1.6732632423543772848170429916717f;
    return lambda * (s >= 0.0f ? s : alpha * __builtin_amdgcn_exp2f(s * 1.44269504088896340736f) - alpha);
}

template <int N>
__device__ __forceinline__ void load_floats(const float* __restrict__ p, float (&v)[N]) {
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

/* the k-th 16-bit entry of a row of the tile-local neighbour table */
__device__ __forceinline__ uint32_t nbl_entry(const v4u& t, int k) {
    const uint32_t w = (k >> 1) == 0 ? t.x : (k >> 1) == 1 ? t.y : (k >> 1) == 2 ? t.z : t.w;
    return (k & 1) ? (w >> 16) : (w & 0xffffu);
}

/* LDS rows: 128-byte rows are XOR-swizzled in 16-byte pieces by the row number, 64- and 16-byte rows lie as they
 * are, other widths get one piece of padding */
__host__ __device__ constexpr bool row_swizzled(int c_in) { return c_in == 32; }
__host__ __device__ constexpr int row_stride(int c_in) { return (c_in == 32 || c_in == 16 || c_in == 4) ? c_in : c_in + 4; }
constexpr int HALO = VMHIP_HALO_MAX;
__host__ __device__ constexpr size_t dma_lds_bytes(int c_in, int c_out, int slots) {
    return (size_t(slots) * (c_in / 4) * ((c_out + 15) / 16) * 64 + size_t((c_out + 15) / 16) * 16 + 2 * size_t(VMHIP_TILE + HALO) * row_stride(c_in)) * 4;
}

template <int C_IN, int C_OUT, int SLOTS, int NW>
__global__ __launch_bounds__(NW * 64, 4) void vm_conv_dma_kernel(VmBatchDev B, VmLayerDev L, const float* __restrict__ in, float* __restrict__ out) {
    constexpr int RB = VMHIP_TILE / (16 * NW);
    static_assert(NW * RB * 16 == VMHIP_TILE, "a block covers one tile");
    static_assert(C_IN % 4 == 0, "rows are staged in 16-byte pieces");
    constexpr int NT = NW * 64;
    constexpr int STEPS = C_IN / 4;
    constexpr int CB = (C_OUT + 15) / 16;
    constexpr int NN = SLOTS - 1;
    static_assert(NN <= VMHIP_NBL_STRIDE, "the tile-local neighbour table holds 8 entries per row");
    constexpr int RS = row_stride(C_IN);
    constexpr bool SWZ = row_swizzled(C_IN);
    constexpr uint32_t FAR_FROM = VMHIP_TILE + HALO;
    constexpr int Q4 = C_IN / 4;  /* data pieces per row */
    constexpr int RSP = RS / 4;   /* pieces per LDS row, padding included */
    constexpr int W_FLOATS = SLOTS * STEPS * CB * 64;
    constexpr int G = STEPS % 4 == 0 ? 4 : STEPS % 2 == 0 ? 2 : 1; /* steps per LDS read */
    constexpr int CH = G; /* steps per pipeline stage (a whole slot per stage measured the same) */
    constexpr int BUF_FLOATS = (VMHIP_TILE + HALO) * RS;
    constexpr int PIECES = (VMHIP_TILE + HALO) * RSP; /* per buffer; a multiple of 64: whole wave loads */
    static_assert(PIECES % 64 == 0, "a buffer is filled by whole wave loads");
    constexpr int N_DMA = (PIECES + NT - 1) / NT;
    constexpr int MAIN_PIECES = VMHIP_TILE * RSP;

    extern __shared__ float4 lds4[];
    float* const w_lds = reinterpret_cast<float*>(lds4);
    float* const b_lds = w_lds + W_FLOATS;
    float* const buf0 = b_lds + CB * 16;
    for (int i = threadIdx.x; i < CB * 16; i += NT) b_lds[i] = i < C_OUT ? L.b[i] : 0.0f;
    for (int i = threadIdx.x; i < W_FLOATS; i += NT) {
        const int e = i % G, l = (i / G) % 64, jg = (i / (G * 64)) % (STEPS / G), cb = (i / (G * 64 * (STEPS / G))) % CB, sl = i / (STEPS * 64 * CB);
        w_lds[i] = reinterpret_cast<const float*>(L.w_mfma)[((sl * STEPS + jg * G + e) * CB + cb) * 64 + l];
    }

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int q = lane >> 4, r16 = lane & 15;
    const int activation = L.activation;

    const int n_tiles = B.n_row_tiles;
    const int xcd = blockIdx.x & 7, lb = blockIdx.x >> 3, gx = gridDim.x >> 3;
    const int per_xcd = (n_tiles + 7) >> 3;
    const int t_end = min(n_tiles, (xcd + 1) * per_xcd);
    int tile = xcd * per_xcd + lb;
    if (tile >= t_end) return; /* the whole block leaves before any barrier or LDS load */
    const int t_last = t_end - 1;

    const uint32_t total_rows = (uint32_t) n_tiles * VMHIP_TILE;
    auto make_rsrc = [](const void* p, uint64_t bytes) {
        return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, (int) (bytes > 0xffffffffull ? 0xffffffffu : (uint32_t) bytes), 0x00020000);
    };
    const __amdgpu_buffer_rsrc_t in_rsrc = make_rsrc(in, (uint64_t) total_rows * C_IN * 4);
    const __amdgpu_buffer_rsrc_t nbl_rsrc = make_rsrc(B.row_nbl, (uint64_t) total_rows * VMHIP_NBL_STRIDE * 2);
    const __amdgpu_buffer_rsrc_t halo_rsrc = make_rsrc(B.tile_halo, (uint64_t) n_tiles * VMHIP_HALO_MAX * 4);
    const __amdgpu_buffer_rsrc_t desc_rsrc = make_rsrc(B.tile_desc, (uint64_t) n_tiles * 16);

    /* Piece p of a buffer = 16 bytes at LDS row p / RSP, position p % RSP. Thread t fills pieces t + k * NT. */
    uint32_t hrow[N_DMA]; /* batch-global row behind the halo pieces this thread fills */
    auto request_halo_rows = [&](int t) {
#pragma unroll
        for (int k = 0; k < N_DMA; ++k) {
            const int p = threadIdx.x + k * NT;
            if ((k + 1) * NT > MAIN_PIECES) { /* compile-time: this k reaches into the halo rows */
                const int h = p / RSP - VMHIP_TILE; /* negative for a main-row piece: out of range, reads 0, unused */
                hrow[k] = __builtin_amdgcn_raw_buffer_load_b32(halo_rsrc, h >= 0 ? (t * VMHIP_HALO_MAX + h) * 4 : 0xffffffffu, 0, 0);
            }
        }
    };
    /* d = {first row, rows in use, halo rows, frame's first row} of the tile, possibly still in vector registers */
    auto stage = [&](const int4& d, float* buf) {
#pragma unroll
        for (int k = 0; k < N_DMA; ++k) {
            if (k * NT + wave * 64 < PIECES) { /* wave-uniform; false only in the last, partial round */
                const int p = threadIdx.x + k * NT;
                const int row_l = p / RSP, cp = p - row_l * RSP;
                const int c = SWZ ? (cp ^ (row_l & 7)) : cp;
                uint32_t off;
                if ((k + 1) * NT <= MAIN_PIECES) {
                    off = (uint32_t) ((d.x + row_l) * Q4 + c) * 16u;
                }
                else {
                    const int h = row_l - VMHIP_TILE;
                    off = h < 0 ? (uint32_t) ((d.x + row_l) * Q4 + c) * 16u : h < d.z ? (hrow[k] * Q4 + c) * 16u : 0xffffffffu;
                }
                if (RSP != Q4 && cp >= Q4) off = 0xffffffffu; /* padding piece */
                __builtin_amdgcn_raw_ptr_buffer_load_lds(in_rsrc, (lds_void*) (buf + (k * NT + wave * 64) * 4), 16, off, 0, 0, 0);
            }
        }
    };
    auto own_row = [&](int rows_in_use, int rb) { return max(0, min(wave * (RB * 16) + rb * 16 + r16, rows_in_use - 1)); };
    auto request_positions = [&](const int4& d, v4u (&nbl)[RB]) {
        if constexpr (NN > 0) {
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) nbl[rb] = vm_load_nbl_row<NN>(nbl_rsrc, (d.x + own_row(d.y, rb)) * (VMHIP_NBL_STRIDE * 2));
        }
    };
    /* descriptors travel through vector memory: a scalar load in flight would turn every LDS wait into a full wait */
    auto load_desc = [&](int t) {
        const v4u d = __builtin_amdgcn_raw_buffer_load_b128(desc_rsrc, t * 16, 0, 0);
        return make_int4((int) d.x, (int) d.y, (int) d.z, (int) d.w);
    };
    auto uniform = [](int4 d) {
        asm volatile("" : "+v"(d.x), "+v"(d.y), "+v"(d.z), "+v"(d.w));
        return make_int4(__builtin_amdgcn_readfirstlane(d.x), __builtin_amdgcn_readfirstlane(d.y), __builtin_amdgcn_readfirstlane(d.z),
                         __builtin_amdgcn_readfirstlane(d.w));
    };
    auto wait_all_loads = [] { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); };

    /* ---- prologue: tiles t and t+1 on their way into the two buffers, t+2 described ---- */
    int t1 = tile + gx, t2 = tile + 2 * gx;
    int4 d_cur = load_desc(tile), d_n1 = load_desc(min(t1, t_last)), d_n2 = load_desc(min(t2, t_last));
    v4u nbl[RB], nbl_n1[RB], nbl_n2[RB];
    request_halo_rows(tile);
    stage(d_cur, buf0); /* waits for the descriptor and the halo row numbers */
    request_positions(d_cur, nbl);
    if (t1 < t_end) {
        request_halo_rows(t1);
        stage(d_n1, buf0 + BUF_FLOATS);
        request_positions(d_n1, nbl_n1);
    }
    request_halo_rows(min(t2, t_last));
    d_cur = uniform(d_cur);
    wait_all_loads();
    __syncthreads(); /* weights, biases and the first tile are in LDS */

    int cur = 0;
    while (true) {
        const float* rows = buf0 + cur * BUF_FLOATS;
        const bool in_use = d_cur.y > 0;
        uint32_t li[RB][SLOTS];
        bool valid[RB];
        bool far = false;
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
            valid[rb] = wave * (RB * 16) + rb * 16 + r16 < d_cur.y;
            li[rb][0] = (uint32_t) own_row(d_cur.y, rb);
#pragma unroll
            for (int s = 0; s < NN; ++s) {
                li[rb][s + 1] = in_use ? nbl_entry(nbl[rb], s) : 0u;
                far |= li[rb][s + 1] >= FAR_FROM;
            }
        }
        const bool any_far = __any(far);

        v4f acc[RB][CB];
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) {
            const v4f bias = *reinterpret_cast<const v4f*>(b_lds + cb * 16 + q * 4);
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) acc[rb][cb] = bias;
        }

        /* matrix work, compiled twice: the usual tile touches nothing but LDS; a tile with not-staged neighbours
         * (wave-uniform choice) patches those lanes' operands from global memory */
        auto contract = [&](auto far_tag) {
            constexpr bool FAR = decltype(far_tag)::value;
            /* a chunk = CH consecutive steps of one slot, fetched G steps per LDS read */
            auto gather = [&](int chunk, float (&x)[RB][CH]) {
                const int sl = chunk / (STEPS / CH), j0 = (chunk % (STEPS / CH)) * CH;
#pragma unroll
                for (int rb = 0; rb < RB; ++rb) {
                    const uint32_t at = (FAR && li[rb][sl] >= FAR_FROM) ? 0u : li[rb][sl];
#pragma unroll
                    for (int j = 0; j < CH; j += G) {
                        float t[G];
                        if constexpr (SWZ) {
                            static_assert(!SWZ || (STEPS == 8 && G == 4), "swizzled rows are 8 pieces of 16 bytes");
                            load_floats<G>(rows + at * RS + (((2 * q + (j0 + j) / G) ^ (at & 7)) << 2), t);
                        }
                        else {
                            load_floats<G>(rows + at * RS + q * STEPS + j0 + j, t);
                        }
#pragma unroll
                        for (int e = 0; e < G; ++e) x[rb][j + e] = t[e];
                    }
                }
                if constexpr (FAR && NN > 0) {
                    if (sl > 0) {
#pragma unroll
                        for (int rb = 0; rb < RB; ++rb) {
                            if (li[rb][sl] >= FAR_FROM) {
                                const int g = B.row_nb[(size_t) (d_cur.x + li[rb][0]) * B.nb_stride + (sl - 1)];
                                load_floats<CH>(in + (size_t) (d_cur.w + g) * C_IN + q * STEPS + j0, x[rb]);
                            }
                        }
                    }
                }
            };
            auto weights = [&](int chunk, float (&a)[CB][CH]) {
                const int sl = chunk / (STEPS / CH), j0 = (chunk % (STEPS / CH)) * CH;
#pragma unroll
                for (int cb = 0; cb < CB; ++cb)
#pragma unroll
                    for (int j = 0; j < CH; j += G) {
                        float t[G];
                        load_floats<G>(w_lds + (((sl * CB + cb) * (STEPS / G) + (j0 + j) / G) * 64 + lane) * G, t);
#pragma unroll
                        for (int e = 0; e < G; ++e) a[cb][j + e] = t[e];
                    }
            };
            /* software pipeline: chunk c+1's operands are requested before chunk c's matrix instructions; the side
             * path runs unpipelined */
            constexpr int CHUNKS = SLOTS * (STEPS / CH);
            constexpr int NBUF = FAR ? 1 : 2;
            float x[NBUF][RB][CH], a[NBUF][CB][CH];
            if constexpr (!FAR) {
                gather(0, x[0]);
                weights(0, a[0]);
            }
#pragma unroll
            for (int c = 0; c < CHUNKS; ++c) {
                const int b = FAR ? 0 : (c & 1);
                if constexpr (FAR) {
                    gather(c, x[0]);
                    weights(c, a[0]);
                }
                else if (c + 1 < CHUNKS) {
                    gather(c + 1, x[b ^ 1]);
                    weights(c + 1, a[b ^ 1]);
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int e = 0; e < CH; ++e)
#pragma unroll
                    for (int cb = 0; cb < CB; ++cb)
#pragma unroll
                        for (int rb = 0; rb < RB; ++rb)
                            acc[rb][cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[b][cb][e], x[b][rb][e], acc[rb][cb], 0, 0, 0);
                if constexpr (FAR) __builtin_amdgcn_sched_barrier(0);
            }
        };
        if (any_far) contract(std::true_type());
        else contract(std::false_type());

        /* ---- the tile's only barrier. Before it: this wave's LDS loads (tile t+1, issued before the matrix loop) are
         * complete. After it: every wave is done reading this buffer and tile t+1 is visible to all. ---- */
        wait_all_loads();
        __syncthreads();

        const bool has_next = t1 < t_end;
        if (t2 < t_end) { /* uniform */
            stage(d_n2, buf0 + cur * BUF_FLOATS); /* tile t+2 into the buffer tile t just left */
            request_positions(d_n2, nbl_n2);
        }
        const int t3 = t2 + gx;
        const int4 d_n3 = load_desc(min(t3, t_last));
        request_halo_rows(min(t3, t_last));
        __builtin_amdgcn_sched_barrier(0);

        /* activation: lane holds channels cb*16 + q*4 + {0..3} of row rb*16 + r16; one uniform branch */
        auto for_each_value = [&](auto fn) {
#pragma unroll
            for (int rb = 0; rb < RB; ++rb)
#pragma unroll
                for (int cb = 0; cb < CB; ++cb)
#pragma unroll
                    for (int v = 0; v < 4; ++v) acc[rb][cb][v] = fn(acc[rb][cb][v]);
        };
        if (activation == VMHIP_SELU) {
            for_each_value([](float v) { return selu(v); });
        }
        else if (activation == VMHIP_RELU) {
            for_each_value([](float v) { return fmaxf(v, 0.0f); });
        }
        else if (activation == VMHIP_TANH) {
            for_each_value([](float v) { return tanhf(v); });
        }
        else {
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) {
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
        }
        /* buffer stores relative to the tile's first output row; lanes without a row get an out-of-range offset */
        const __amdgpu_buffer_rsrc_t out_rsrc = make_rsrc(out + (size_t) d_cur.x * C_OUT, (uint64_t) VMHIP_TILE * C_OUT * 4);
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
#pragma unroll
            for (int cb = 0; cb < CB; ++cb) {
                const int o = cb * 16 + q * 4;
                const uint32_t at = (li[rb][0] * C_OUT + o) * 4;
                if constexpr (C_OUT % 4 == 0) {
                    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4u, acc[rb][cb]), out_rsrc, (valid[rb] && o < C_OUT) ? at : 0xffffffffu, 0, 0);
                }
                else {
#pragma unroll
                    for (int v = 0; v < 4; ++v)
                        if (cb * 16 + v < C_OUT)
                            __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(acc[rb][cb][v]), out_rsrc,
                                                                  (valid[rb] && o + v < C_OUT) ? at + v * 4 : 0xffffffffu, 0, 0);
                }
            }
        }

        if (!has_next) break;
        /* rotate: t+1 becomes current */
        d_cur = uniform(d_n1);
        d_n1 = d_n2;
        d_n2 = d_n3;
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) nbl[rb] = nbl_n1[rb], nbl_n1[rb] = nbl_n2[rb];
        tile = t1;
        t1 = t2;
        t2 = t3;
        cur ^= 1;
    }
    wait_all_loads(); /* no LDS load may outlive the wave */
}

template <int C_IN, int C_OUT, int SLOTS>
int launch_dma(const VmBatchDev& B, const VmLayerDev& L, const float* in, float* out, hipStream_t stream) {
    constexpr size_t lds = dma_lds_bytes(C_IN, C_OUT, SLOTS);
    static_assert(lds <= 160 * 1024, "weights and two row buffers must fit the CU's LDS");
    /* the kernel addresses its input rows with 32-bit byte offsets */
    if ((uint64_t) B.n_row_tiles * VMHIP_TILE * C_IN * 4 > 0xffffffffull) return -1;
    constexpr bool single = 2 * lds > 160 * 1024; /* one block of 16 waves, else two (or more) of 8 */
    constexpr int NW = single ? 16 : 8;
    auto kernel = vm_conv_dma_kernel<C_IN, C_OUT, SLOTS, NW>;
    static std::atomic<bool> configured{false}; /* engines on several host threads may get here together */
    if (!configured) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, int(lds)) != hipSuccess) {
            (void) hipGetLastError();
            return -1;
        }
        configured = true;
    }
    int per_cu = single ? 1 : 2;
    if (const char* e = getenv("VMHIP_LDS_BLOCKS_PER_CU")) per_cu = atoi(e) > 0 ? atoi(e) : per_cu;
    int grid = 256 * per_cu;
    const int need = ((B.n_row_tiles + 7) / 8) * 8;
    if (grid > need) grid = need;
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(NW * 64), lds, stream, B, L, in, out);
    return 0;
}

}  // namespace

#define VM_FOR_EACH_DMA_SHAPE(X) \
    X(4, 16, 7)                  \
    X(16, 16, 7)                 \
    X(16, 32, 7)                 \
    X(32, 32, 7)                 \
    X(32, 16, 7)                 \
    X(16, 3, 7)                  \
    X(16, 2, 7)                  \
    X(4, 64, 7)                  \
    X(4, 24, 9)                  \
    X(24, 24, 9)                 \
    X(24, 4, 9)                  \
    /* the reference's example network: 4->16, 16->16 x5, 16->8, 8->8 x5, 8->5 */ \
    X(16, 8, 7)                  \
    X(8, 8, 7)                   \
    X(8, 5, 7)

bool vm_dma_supported(int c_in, int c_out, int slots) {
#define X(CI, CO, SL) \
    if (c_in == CI && c_out == CO && slots == SL) return true;
    VM_FOR_EACH_DMA_SHAPE(X)
#undef X
    return false;
}

int vm_launch_conv_dma(const VmBatchDev& B, const VmLayerDev& L, const float* in, float* out, hipStream_t stream, const char** kernel_name) {
    if (B.n_row_tiles <= 0) return 0;
    if (!B.row_nbl || !B.tile_halo || !B.tile_desc || !L.w_mfma || L.in_bf16 || L.out_bf16 || L.arith_bf16) return -1;
#define X(CI, CO, SL)                                                    \
    if (L.c_in == CI && L.c_out == CO && L.slots == SL) {                \
        if (kernel_name) *kernel_name = "conv_dma_" #CI "x" #CO "s" #SL; \
        return launch_dma<CI, CO, SL>(B, L, in, out, stream);            \
    }
    VM_FOR_EACH_DMA_SHAPE(X)
#undef X
    return -1;
}

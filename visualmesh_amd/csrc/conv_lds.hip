/*
 * conv_lds.hip - graph-convolution layers on the matrix cores with both operands fed from LDS: neighbour gather +
 * dense + bias + activation in one kernel (reference engine/cpu/engine.hpp:213-264, apply_activation.hpp:34-84).
 *
 * The contraction and the operand layout are those of conv_mfma.hip (v_mfma_f32_16x16x4_f32, lane group q takes
 * the q-th quarter of every gathered row, weights stored in consumption order). What differs is where the
 * gathered rows come from. A row tile's sources are its own 256 rows plus about 100 distinct rows of other tiles
 * (tile_halo, at most VMHIP_HALO_MAX), and row_nbl names every neighbour as a position in that list. So a block
 *   1. copies the tile's rows (one contiguous run of global memory) and its halo rows into LDS with coalesced
 *      16-byte loads: every row is requested once per tile instead of once per gather slot;
 *   2. gathers matrix operands from LDS with ds_read, the weights next to them: no vector-memory instruction
 *      sits between the matrix instructions, which is what held the register-gather kernel near 57 % of the
 *      matrix peak;
 *   3. applies the activation and writes the output rows.
 * The global loads of tile t+1 (rows, halo rows, neighbour positions) are issued before the matrix work of tile
 * t and land in registers; they are written to LDS after the barrier that ends tile t. Halo row numbers and tile
 * descriptors are requested two tiles ahead because the row loads depend on them.
 *
 * A kernel stages as many halo rows as its LDS budget allows (144 to 256 depending on the layer shape). A
 * neighbour beyond that, or marked VMHIP_NBL_FAR in row_nbl, is not staged: a wave that holds such an entry
 * takes a side path that reads that row from global memory (a few per cent of the tiles of the benchmark
 * meshes have more than 144 halo rows).
 *
 * Blocks are persistent and XCD aware exactly as in conv_mfma.hip.
 */
#include <cstdlib>
#include <type_traits>

#include <atomic>

#include "vmhip_internal.h"

namespace {

typedef float v4f __attribute__((ext_vector_type(4)));

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

/* N consecutive floats with the widest loads their count allows (the caller guarantees matching alignment) */
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
typedef uint32_t v4u32 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint32_t nbl_entry(const v4u32& t, int k) {
    const uint32_t w = (k >> 1) == 0 ? t.x : (k >> 1) == 1 ? t.y : (k >> 1) == 2 ? t.z : t.w;
    return (k & 1) ? (w >> 16) : (w & 0xffffu);
}

/* How staged rows are spread over the LDS banks. 128-byte rows (C_IN = 32) keep their size and XOR the position
 * of each 16-byte piece with the low bits of the row number; 64-byte and 16-byte rows need nothing (consecutive
 * rows already rotate through the banks); other widths get 16 bytes of padding per row. */
__host__ __device__ constexpr bool row_swizzled(int c_in) { return c_in == 32; }
__host__ __device__ constexpr int row_stride(int c_in) { return (c_in == 32 || c_in == 16 || c_in == 4) ? c_in : c_in + 4; }
__host__ __device__ constexpr size_t lds_bytes(int c_in, int c_out, int slots, int halo) {
    return (size_t(slots) * (c_in / 4) * ((c_out + 15) / 16) * 64 + size_t((c_out + 15) / 16) * 16 + size_t(VMHIP_TILE + halo) * row_stride(c_in)) * 4;
}
/* Halo rows a block stages: all VMHIP_HALO_MAX if two blocks then still fit a CU's 160 KB of LDS (two blocks
 * overlap one's activation/store/staging phase with the other's matrix work), else 192 or 128
 * if that lets two fit, else everything in one block per CU. */
__host__ __device__ constexpr int halo_rows(int c_in, int c_out, int slots) {
    for (int h = VMHIP_HALO_MAX; h >= 128; h -= 64)
        if (2 * lds_bytes(c_in, c_out, slots, h) <= 160 * 1024) return h;
    return VMHIP_HALO_MAX;
}

/* NW waves per block, RB row blocks of 16 rows per wave: NW * RB * 16 == VMHIP_TILE. */
/* C_OUT_T > 0: that many output channels, known to the compiler. C_OUT_T < 0: -C_OUT_T column blocks of 16 and the
 * layer's own count of output channels (L.c_out, at most 16 per block) read at run time - the instantiations that
 * take every shape the enumerated ones leave out. */
template <int C_IN, int C_OUT_T, int SLOTS, int NW, int HALO, int OUT_FMT>
__global__ __launch_bounds__(NW * 64, 4) void vm_conv_lds_kernel(VmBatchDev B, VmLayerDev L, const float* __restrict__ in, float* __restrict__ out) {
    static_assert(OUT_FMT == VM_ROWS_F32 || (OUT_FMT == VM_ROWS_BF16X2 && C_OUT_T > 0 && C_OUT_T % 16 == 0), "rows go out as fp32, or as hi + lo pairs of bf16 for a bf16 layer to read");
    constexpr bool ANY_WIDTH = C_OUT_T < 0;
    const int C_OUT = ANY_WIDTH ? L.c_out : C_OUT_T;
    constexpr int RB = VMHIP_TILE / (16 * NW);
    static_assert(NW * RB * 16 == VMHIP_TILE, "a block covers one tile");
    static_assert(C_IN % 4 == 0, "rows are staged in 16-byte pieces");
    constexpr int NT = NW * 64;
    constexpr int STEPS = C_IN / 4; /* matrix steps per slot = floats in a lane's quarter row */
    constexpr int CB = ANY_WIDTH ? -C_OUT_T : (C_OUT_T + 15) / 16;
    constexpr int NN = SLOTS - 1;
    static_assert(NN <= VMHIP_NBL_STRIDE, "the tile-local neighbour table holds 8 entries per row");
    constexpr int RS = row_stride(C_IN);
    constexpr bool SWZ = row_swizzled(C_IN);
    constexpr uint32_t FAR_FROM = VMHIP_TILE + HALO; /* positions from here on are not staged by this kernel */
    constexpr int Q4 = C_IN / 4; /* 16-byte pieces per row */
    constexpr int W_FLOATS = SLOTS * STEPS * CB * 64;
    constexpr int G = STEPS % 4 == 0 ? 4 : STEPS % 2 == 0 ? 2 : 1; /* weights fetched per LDS read */
    constexpr int N_MAIN = (VMHIP_TILE * Q4 + NT - 1) / NT;      /* pieces of the tile's rows per thread */
    constexpr int N_HALO = (HALO * Q4 + NT - 1) / NT;  /* pieces of halo rows per thread */

    extern __shared__ float4 lds4[];
    float* const w_lds = reinterpret_cast<float*>(lds4);
    float* const b_lds = w_lds + W_FLOATS; /* CB * 16 biases, zero for padded channels */
    float* const rows = b_lds + CB * 16;
    for (int i = threadIdx.x; i < CB * 16; i += NT) b_lds[i] = i < C_OUT ? L.b[i] : 0.0f;
    /* Weights: global order is [slot][step][column block][lane]; in LDS a lane's G consecutive steps sit together,
     * [slot][column block][step / G][lane][G], so that one ds_read fetches G of them. */
    for (int i = threadIdx.x; i < W_FLOATS; i += NT) {
        const int e = i % G, l = (i / G) % 64, jg = (i / (G * 64)) % (STEPS / G), cb = (i / (G * 64 * (STEPS / G))) % CB, sl = i / (STEPS * 64 * CB);
        w_lds[i] = reinterpret_cast<const float*>(L.w_mfma)[((sl * STEPS + jg * G + e) * CB + cb) * 64 + l];
    }

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int q = lane >> 4, r16 = lane & 15;
    const int activation = L.activation;

    const int n_tiles = vm_row_tiles(B);
    const int xcd = blockIdx.x & 7, lb = blockIdx.x >> 3, gx = gridDim.x >> 3;
    const int per_xcd = (n_tiles + 7) >> 3;
    const int t_end = min(n_tiles, (xcd + 1) * per_xcd);
    int tile = xcd * per_xcd + lb;
    if (tile >= t_end) return; /* the whole block leaves: no barrier is left waiting */

    /* ---- staging: thread-private pieces of the next tile ----
     * Every global read of the tile loop is an unconditional buffer load with a 32-bit offset: out-of-range
     * offsets (stale halo entries, tiles past the end) read zeros instead of faulting, so there are no branches
     * around the loads and the compiler can wait for exactly the loads it needs (vector-memory operations retire
     * in order; a branch would force it to wait for all of them, stores included). */
    typedef uint32_t v4u __attribute__((ext_vector_type(4)));
    const uint32_t total_rows = (uint32_t) n_tiles * VMHIP_TILE;
    auto make_rsrc = [](const void* p, uint64_t bytes) {
        return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, (int) (bytes > 0xffffffffull ? 0xffffffffu : (uint32_t) bytes), 0x00020000);
    };
    const __amdgpu_buffer_rsrc_t in_rsrc = make_rsrc(in, (uint64_t) total_rows * C_IN * 4);
    const __amdgpu_buffer_rsrc_t nbl_rsrc = make_rsrc(B.row_nbl, (uint64_t) total_rows * VMHIP_NBL_STRIDE * 2);
    const __amdgpu_buffer_rsrc_t halo_rsrc = make_rsrc(B.tile_halo, (uint64_t) n_tiles * VMHIP_HALO_MAX * 4);
    const __amdgpu_buffer_rsrc_t desc_rsrc = make_rsrc(B.tile_desc, (uint64_t) n_tiles * 16);

    v4u st_main[N_MAIN], st_halo[N_HALO];
    uint32_t hrow[N_HALO];
    auto request_halo_rows = [&](int t) {
#pragma unroll
        for (int k = 0; k < N_HALO; ++k) {
            const int h = (threadIdx.x + k * NT) / Q4; /* entries past the tile's count are stale and unused */
            hrow[k] = __builtin_amdgcn_raw_buffer_load_b32(halo_rsrc, (t * VMHIP_HALO_MAX + h) * 4, 0, 0);
        }
    };
    /* d = {first row, rows in use, halo rows, frame's first row}, still in vector registers */
    auto request_rows = [&](const int4& d) {
#pragma unroll
        for (int k = 0; k < N_MAIN; ++k) st_main[k] = __builtin_amdgcn_raw_buffer_load_b128(in_rsrc, (d.x * Q4 + (int) threadIdx.x + k * NT) * 16, 0, 0);
#pragma unroll
        for (int k = 0; k < N_HALO; ++k) {
            const int idx = threadIdx.x + k * NT;
            const int h = idx / Q4, c = idx % Q4;
            /* slots past the tile's halo count: an out-of-range offset reads zeros without touching memory */
            st_halo[k] = __builtin_amdgcn_raw_buffer_load_b128(in_rsrc, h < d.z ? (hrow[k] * Q4 + c) * 16 : 0xffffffffu, 0, 0);
        }
    };
    auto write_rows = [&]() {
        v4u* rows4 = reinterpret_cast<v4u*>(rows);
#pragma unroll
        for (int k = 0; k < N_MAIN; ++k) {
            const int idx = threadIdx.x + k * NT;
            const int r = idx / Q4, c = idx - r * Q4;
            if (N_MAIN * NT == VMHIP_TILE * Q4 || idx < VMHIP_TILE * Q4) rows4[(r * RS) / 4 + (SWZ ? (c ^ (r & 7)) : c)] = st_main[k];
        }
#pragma unroll
        for (int k = 0; k < N_HALO; ++k) {
            const int idx = threadIdx.x + k * NT;
            const int h = idx / Q4, c = idx - h * Q4;
            if (N_HALO * NT == HALO * Q4 || h < HALO) rows4[((VMHIP_TILE + h) * RS) / 4 + (SWZ ? (c ^ (h & 7)) : c)] = st_halo[k];
        }
    };
    /* the lane's rows of a tile: rows past the tile's count compute on its last row (the frame's null row) and
     * skip the store */
    auto own_row = [&](int rows_in_use, int rb) { return max(0, min(wave * (RB * 16) + rb * 16 + r16, rows_in_use - 1)); };
    auto request_positions = [&](const int4& d, v4u (&nbl)[RB]) {
        if constexpr (NN > 0) {
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) nbl[rb] = vm_load_nbl_row<NN>(nbl_rsrc, (d.x + own_row(d.y, rb)) * (VMHIP_NBL_STRIDE * 2));
        }
    };
    /* Tile descriptors are wave-uniform but must not be fetched with scalar loads: scalar loads return out of
     * order on the counter that LDS reads use too, so one descriptor in flight would turn every LDS wait of the
     * matrix loop into a wait for that (global-latency) load. */
    auto load_desc = [&](int t) {
        const v4u d = __builtin_amdgcn_raw_buffer_load_b128(desc_rsrc, t * 16, 0, 0);
        return make_int4((int) d.x, (int) d.y, (int) d.z, (int) d.w);
    };
    /* to scalar registers; the empty asm keeps the compiler from doing this (and so waiting for the load) early */
    auto uniform = [](int4 d) {
        asm volatile("" : "+v"(d.x), "+v"(d.y), "+v"(d.z), "+v"(d.w));
        return make_int4(__builtin_amdgcn_readfirstlane(d.x), __builtin_amdgcn_readfirstlane(d.y), __builtin_amdgcn_readfirstlane(d.z),
                         __builtin_amdgcn_readfirstlane(d.w));
    };

    /* ---- prologue: everything tile `tile` needs, then the look-ahead for the next one. Tiles past the end of
     * the block's share are clamped to its last tile: their loads are redundant, never wrong. ---- */
    const int t_last = t_end - 1;
    int4 d_cur = uniform(load_desc(tile));
    int next = tile + gx;
    v4u nbl[RB], nbl_next[RB];
    request_halo_rows(tile);
    request_rows(d_cur);
    request_positions(d_cur, nbl);
    int4 d_next = load_desc(min(next, t_last)), d_after = d_next;
    request_halo_rows(min(next, t_last));
    while (true) {
        write_rows();
        __syncthreads(); /* rows (and, the first time, weights) are in LDS */

        const bool has_next = next < t_end;
        const int after = next + gx;
        request_rows(d_next);
        d_after = load_desc(min(after, t_last));
        request_halo_rows(min(after, t_last));
        __builtin_amdgcn_sched_barrier(0);

        {
            /* an empty tile (no rows in use) runs the same code on position 0 and stores nothing */
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

            /* The matrix work, compiled twice: the usual tile touches nothing but LDS here; a tile with
             * not-staged neighbours (wave-uniform choice) patches those lanes' operands from global memory. */
            auto contract = [&](auto far_tag) {
                constexpr bool FAR = decltype(far_tag)::value;
                /* chunk = G consecutive steps of one slot: the lane's G inputs per row block ... */
                auto gather = [&](int chunk, float (&x)[RB][G]) {
                    const int sl = chunk / (STEPS / G), jg = chunk % (STEPS / G);
#pragma unroll
                    for (int rb = 0; rb < RB; ++rb) {
                        const uint32_t at = (FAR && li[rb][sl] >= FAR_FROM) ? 0u : li[rb][sl];
                        if constexpr (SWZ) {
                            /* the lane's quarter row is pieces 2q and 2q+1, each moved by the row's low bits */
                            static_assert(STEPS == 8 && G == 4, "swizzled rows are 8 pieces of 16 bytes");
                            load_floats<G>(rows + at * RS + (((2 * q + jg) ^ (at & 7)) << 2), x[rb]);
                        }
                        else {
                            load_floats<G>(rows + at * RS + q * STEPS + jg * G, x[rb]);
                        }
                    }
                    if constexpr (FAR && NN > 0) {
                        if (sl > 0) {
#pragma unroll
                            for (int rb = 0; rb < RB; ++rb) {
                                if (li[rb][sl] >= FAR_FROM) {
                                    const int g = B.row_nb[(size_t) (d_cur.x + li[rb][0]) * B.nb_stride + (sl - 1)];
                                    load_floats<G>(in + (size_t) (d_cur.w + g) * C_IN + q * STEPS + jg * G, x[rb]);
                                }
                            }
                        }
                    }
                };
                /* ... and the weights of those steps, all column blocks */
                auto weights = [&](int chunk, float (&a)[CB][G]) {
                    const int sl = chunk / (STEPS / G), jg = chunk % (STEPS / G);
#pragma unroll
                    for (int cb = 0; cb < CB; ++cb) load_floats<G>(w_lds + (((sl * CB + cb) * (STEPS / G) + jg) * 64 + lane) * G, a[cb]);
                };
                /* Software pipeline: chunk c+1's operands are requested before chunk c's matrix instructions. The
                 * side path runs unpipelined: it is rare, and its extra address registers would otherwise push the
                 * staged rows of the next tile out of the register file. */
                constexpr int CHUNKS = SLOTS * (STEPS / G);
                constexpr int NBUF = FAR ? 1 : 2;
                /* weights are double-buffered only where registers allow (16 accumulator registers leave no room) */
                constexpr int ABUF = (FAR || RB * CB * 4 >= 16) ? 1 : 2;
                float x[NBUF][RB][G], a[ABUF][CB][G];
                if constexpr (!FAR) {
                    gather(0, x[0]);
                    if constexpr (ABUF == 2) weights(0, a[0]);
                }
#pragma unroll
                for (int c = 0; c < CHUNKS; ++c) {
                    const int cur = FAR ? 0 : (c & 1);
                    const int acur = ABUF == 2 ? (c & 1) : 0;
                    if constexpr (FAR) {
                        gather(c, x[0]);
                    }
                    else if (c + 1 < CHUNKS) {
                        gather(c + 1, x[cur ^ 1]);
                    }
                    if constexpr (ABUF == 1) {
                        weights(c, a[0]);
                    }
                    else if (c + 1 < CHUNKS) {
                        weights(c + 1, a[acur ^ 1]);
                    }
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int e = 0; e < G; ++e)
#pragma unroll
                        for (int cb = 0; cb < CB; ++cb)
#pragma unroll
                            for (int rb = 0; rb < RB; ++rb)
                                acc[rb][cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[acur][cb][e], x[cur][rb][e], acc[rb][cb], 0, 0, 0);
                    if constexpr (FAR || ABUF == 1) __builtin_amdgcn_sched_barrier(0);
                }
            };
            if (any_far) contract(std::true_type());
            else contract(std::false_type());
            /* the next tile's neighbour positions: requested only now, when the operand registers are free */
            request_positions(d_next, nbl_next);

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
                for_each_value([](float a) { return selu(a); });
            }
            else if (activation == VMHIP_RELU) {
                for_each_value([](float a) { return fmaxf(a, 0.0f); });
            }
            else if (activation == VMHIP_TANH) {
                for_each_value([](float a) { return tanhf(a); });
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
            /* buffer stores relative to the tile's first output row; lanes without a row get an out-of-range
             * offset, which the hardware drops: no branch around the stores either */
            const __amdgpu_buffer_rsrc_t out_rsrc = make_rsrc(out + (size_t) d_cur.x * C_OUT, (uint64_t) VMHIP_TILE * C_OUT * 4);
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) {
                if constexpr (OUT_FMT == VM_ROWS_BF16X2) {
                    /* hi = bf16(x), lo = bf16(x - hi), the difference being exact; C_OUT hi values, then C_OUT lo values.
                     * The host has ordered this layer's output columns so that matrix column cb * 16 + q * 4 + v is channel
                     * q * 4 * CB + cb * 4 + v: a lane's 4 * CB values are neighbours in the row and leave as 16-byte stores,
                     * four lanes filling a row's 128-byte plane (with the columns in their own order a lane's pieces were
                     * 8 bytes, 32 bytes apart, in twice as many store instructions: 3.6 ms instead of 2.9 for the 4 -> 64
                     * layer of a 64-frame batch; fp32 rows take 2.6). */
                    static_assert(CB % 2 == 0, "a lane's hi (lo) values are whole 16-byte pieces");
                    typedef __bf16 v2bf __attribute__((ext_vector_type(2)));
                    auto pack = [](float a, float b) {
                        v2bf t;
                        t[0] = (__bf16) a, t[1] = (__bf16) b;
                        return __builtin_bit_cast(uint32_t, t);
                    };
                    uint32_t hi[CB][2], lo[CB][2];
#pragma unroll
                    for (int cb = 0; cb < CB; ++cb) {
                        const v4f x = acc[rb][cb];
                        hi[cb][0] = pack(x[0], x[1]), hi[cb][1] = pack(x[2], x[3]);
                        lo[cb][0] = pack(x[0] - __uint_as_float(hi[cb][0] << 16), x[1] - __uint_as_float(hi[cb][0] & 0xffff0000u));
                        lo[cb][1] = pack(x[2] - __uint_as_float(hi[cb][1] << 16), x[3] - __uint_as_float(hi[cb][1] & 0xffff0000u));
                    }
                    const uint32_t at2 = li[rb][0] * (C_OUT * 4) + q * (CB * 8);
#pragma unroll
                    for (int p = 0; p < CB / 2; ++p) {
                        const v4u h4 = {hi[2 * p][0], hi[2 * p][1], hi[2 * p + 1][0], hi[2 * p + 1][1]};
                        const v4u l4 = {lo[2 * p][0], lo[2 * p][1], lo[2 * p + 1][0], lo[2 * p + 1][1]};
                        __builtin_amdgcn_raw_buffer_store_b128(h4, out_rsrc, valid[rb] ? at2 + p * 16 : 0xffffffffu, 0, 0);
                        __builtin_amdgcn_raw_buffer_store_b128(l4, out_rsrc, valid[rb] ? at2 + p * 16 + C_OUT * 2 : 0xffffffffu, 0, 0);
                    }
                    continue;
                }
#pragma unroll
                for (int cb = 0; cb < CB; ++cb) {
                    const int o = cb * 16 + q * 4;
                    const uint32_t at = (li[rb][0] * C_OUT + o) * 4;
                    if constexpr (!ANY_WIDTH && C_OUT_T % 4 == 0) {
                        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4u, acc[rb][cb]), out_rsrc, (valid[rb] && o < C_OUT) ? at : 0xffffffffu, 0, 0);
                    }
                    else if (ANY_WIDTH && C_OUT % 4 == 0) { /* one uniform branch for the whole kernel: rows are whole 16-byte pieces */
                        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4u, acc[rb][cb]), out_rsrc, (valid[rb] && o < C_OUT) ? at : 0xffffffffu, 0, 0);
                    }
                    else {
#pragma unroll
                        for (int v = 0; v < 4; ++v)
                            if (ANY_WIDTH || cb * 16 + v < C_OUT_T) /* known width: some lane group holds a real channel here */
                                __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(acc[rb][cb][v]), out_rsrc,
                                                                      (valid[rb] && o + v < C_OUT) ? at + v * 4 : 0xffffffffu, 0, 0);
                    }
                }
            }
        }
        if (!has_next) break;
        __syncthreads(); /* every wave is done reading this tile's rows */
        d_cur = uniform(d_next);
        d_next = d_after;
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) nbl[rb] = nbl_next[rb];
        tile = next;
        next = after;
    }
}

template <int C_IN, int C_OUT_T, int SLOTS, int OUT_FMT = VM_ROWS_F32>
int launch_lds(const VmBatchDev& B, const VmLayerDev& L, const float* in, float* out, hipStream_t stream) {
    constexpr int C_OUT = C_OUT_T > 0 ? C_OUT_T : -16 * C_OUT_T; /* what the LDS is sized for */
    constexpr int HALO = halo_rows(C_IN, C_OUT, SLOTS);
    constexpr size_t lds = lds_bytes(C_IN, C_OUT, SLOTS, HALO);
    static_assert(lds <= 160 * 1024, "weights and staged rows must fit the CU's LDS");
    /* the kernel addresses its input rows with 32-bit byte offsets */
    if ((uint64_t) B.n_row_tiles * VMHIP_TILE * C_IN * 4 > 0xffffffffull) return -1;
    /* Two or more blocks of 8 waves per CU where LDS allows (registers are capped at 128 per lane, four waves
     * per SIMD); otherwise one block of 16 waves. */
    constexpr bool single = 2 * lds > 160 * 1024;
    constexpr int NW = single ? 16 : 8;
    auto kernel = vm_conv_lds_kernel<C_IN, C_OUT_T, SLOTS, NW, HALO, OUT_FMT>;
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

#define VM_FOR_EACH_LDS_SHAPE(X) \
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

/* ... and the shapes that can also write their rows as hi + lo pairs of bf16 */
#define VM_FOR_EACH_LDS_SPLIT_SHAPE(X) \
    X(4, 64, 7)

/* Every other shape with input rows of whole 16-byte pieces up to 32 channels and up to 64 output channels runs on
 * instantiations that know the input width and the number of 16-channel column blocks, and read the exact number of
 * output channels at run time (reference engine/opencl/operation/make_network.hpp:43-214 generates a kernel for any
 * shape). X(C_in, column blocks, slots). */
/* 7 and 9 gather slots: the six- and eight-neighbour models (Ring6, NMGrid8 ...); 5: the four-neighbour ones
 * (reference model/ring4.hpp, xygrid4.hpp, xmgrid4.hpp, nmgrid4.hpp) */
#define VM_LDS_ANY_WIDTHS(X, CI) X(CI, 1, 7) X(CI, 2, 7) X(CI, 3, 7) X(CI, 4, 7) X(CI, 1, 9) X(CI, 2, 9) X(CI, 3, 9) X(CI, 4, 9) X(CI, 1, 5) X(CI, 2, 5) X(CI, 3, 5) X(CI, 4, 5)
#define VM_FOR_EACH_LDS_ANY_SHAPE(X) \
    VM_LDS_ANY_WIDTHS(X, 4)          \
    VM_LDS_ANY_WIDTHS(X, 8)          \
    VM_LDS_ANY_WIDTHS(X, 12)         \
    VM_LDS_ANY_WIDTHS(X, 16)         \
    VM_LDS_ANY_WIDTHS(X, 20)         \
    VM_LDS_ANY_WIDTHS(X, 24)         \
    VM_LDS_ANY_WIDTHS(X, 28)         \
    VM_LDS_ANY_WIDTHS(X, 32)

bool vm_lds_supported(int c_in, int c_out, int slots, int out_fmt) {
#define X(CI, CO, SL) \
    if (c_in == CI && c_out == CO && slots == SL) return true;
    if (out_fmt == VM_ROWS_F32) {
        VM_FOR_EACH_LDS_SHAPE(X)
        return c_in % 4 == 0 && c_in >= 4 && c_in <= 32 && c_out >= 1 && c_out <= 64 && (slots == 5 || slots == 7 || slots == 9);
    }
    else if (out_fmt == VM_ROWS_BF16X2) {
        VM_FOR_EACH_LDS_SPLIT_SHAPE(X)
    }
#undef X
    return false;
}

int vm_launch_conv_lds(const VmBatchDev& B, const VmLayerDev& L, const float* in, float* out, hipStream_t stream, const char** kernel_name) {
    if (B.n_row_tiles <= 0) return 0;
    if (!B.row_nbl || !B.tile_halo || !B.tile_desc || !L.w_mfma || L.in_bf16 || L.arith_bf16) return -1;
    if (L.out_bf16 == VM_ROWS_BF16X2) {
#define X(CI, CO, SL)                                                          \
    if (L.c_in == CI && L.c_out == CO && L.slots == SL) {                      \
        if (kernel_name) *kernel_name = "conv_lds_tox2_" #CI "x" #CO "s" #SL;  \
        return launch_lds<CI, CO, SL, VM_ROWS_BF16X2>(B, L, in, out, stream);  \
    }
        VM_FOR_EACH_LDS_SPLIT_SHAPE(X)
#undef X
        return -1;
    }
    if (L.out_bf16) return -1;
#define X(CI, CO, SL)                                                       \
    if (L.c_in == CI && L.c_out == CO && L.slots == SL) {                   \
        if (kernel_name) *kernel_name = "conv_lds_" #CI "x" #CO "s" #SL;    \
        return launch_lds<CI, CO, SL>(B, L, in, out, stream);               \
    }
    VM_FOR_EACH_LDS_SHAPE(X)
#undef X
    const int blocks = (L.c_out + 15) / 16;
#define X(CI, CBL, SL)                                                                       \
    if (L.c_in == CI && blocks == CBL && L.slots == SL) {                                    \
        if (kernel_name) *kernel_name = vm_kernel_name("conv_lds", L.c_in, L.c_out, L.slots); \
        return launch_lds<CI, -CBL, SL>(B, L, in, out, stream);                              \
    }
    VM_FOR_EACH_LDS_ANY_SHAPE(X)
#undef X
    return -1;
}

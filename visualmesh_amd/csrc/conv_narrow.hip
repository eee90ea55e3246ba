/*
 * conv_narrow.hip - graph-convolution layers with at most four output channels (the class layers: 16 -> 3,
 * 16 -> 2, 24 -> 4) on the matrix cores without padding the output to 16 columns: neighbour gather + dense + bias
 * + activation in one kernel (reference engine/cpu/engine.hpp:213-264, apply_activation.hpp:34-84).
 *
 * v_mfma_f32_4x4x1_16b_f32 multiplies sixteen independent 4x1 by 1x4 blocks: with the weights as A (lane l supplies
 * W[k][l % 4], the same for every block) and one input value per lane as B (lane l supplies in[src(row l)][k]),
 * a wave computes 64 rows x 4 output channels per instruction and reduction step, and lane l ends up holding the
 * four output channels of row l: the activation (softmax included) needs no cross-lane traffic and the row is
 * written with one store. Per row that is 8 matrix-pipe cycles for every 64 x 4 x 1 products: no waste against
 * the 16-column instruction, which spends 5.3 times more on a 3-channel layer.
 *
 * Staging follows conv_flow.hip: rows travel from global memory straight into LDS (buffer_load ... lds), tile-local tables, XCD-aware persistent tile walk, a side path for
 * neighbours that are not staged. A lane reads its whole source row from LDS per gather slot, a quarter at a time.
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

/* LDS rows: a lane reads piece c of its own source row, all lanes of an instruction the same c. A 64-byte row
 * (C_IN = 16) spans 16 of the 64 banks, so row r, piece c lies in the four banks 16 (r % 4) + 4 c: with the pieces
 * left where they are, sixteen lanes would meet in four groups of banks. The pieces are therefore XORed with bits
 * 2 and 3 of the row number: sixteen consecutive rows then reach sixteen different groups (XORing with bits 0 and
 * 1, which already choose the quarter of the banks, leaves the four-way conflict: 35 us against 31 us on 16 -> 3).
 * Other widths get one piece of padding, which rotates consecutive rows through the banks by itself. */
__host__ __device__ constexpr bool row_swizzled(int c_in) { return c_in == 16; }
__host__ __device__ constexpr int row_stride(int c_in) { return c_in == 16 ? c_in : c_in + 4; }
constexpr int HALO = VMHIP_HALO_MAX;
constexpr int NW = 4; /* 64 rows per wave */
/* Row buffers per block. One, with up to four blocks of four waves sharing a CU (each meets its next tile at the top
 * of its loop while the others work), measured faster than two buffers and two blocks per CU: 28 us against 31 us
 * on 16 -> 3. */
constexpr int NBUFS = 1;
__host__ __device__ constexpr size_t narrow_lds_bytes(int c_in, int slots) {
    return (size_t(slots) * c_in * 4 + 4 + NBUFS * size_t(VMHIP_TILE + HALO) * row_stride(c_in)) * 4;
}

template <int C_IN, int C_OUT, int SLOTS>
__global__ __launch_bounds__(NW * 64) void vm_conv_narrow_kernel(VmBatchDev B, VmLayerDev L, const float* __restrict__ in, float* __restrict__ out) {
    static_assert(C_OUT >= 1 && C_OUT <= 4, "one 4x4x1 block holds at most four output channels");
    static_assert(C_IN % 4 == 0, "rows are staged in 16-byte pieces");
    constexpr int NT = NW * 64;
    static_assert(NT == VMHIP_TILE, "one lane per row of the tile");
    constexpr int NN = SLOTS - 1;
    static_assert(NN <= VMHIP_NBL_STRIDE, "the tile-local neighbour table holds 8 entries per row");
    constexpr int RS = row_stride(C_IN);
    constexpr bool SWZ = row_swizzled(C_IN);
    constexpr uint32_t FAR_FROM = VMHIP_TILE + HALO;
    constexpr int Q4 = C_IN / 4;  /* data pieces per row */
    constexpr int RSP = RS / 4;   /* pieces per LDS row, padding included */
    constexpr int W_FLOATS = SLOTS * C_IN * 4;
    constexpr int BUF_FLOATS = (VMHIP_TILE + HALO) * RS;
    constexpr int PIECES = (VMHIP_TILE + HALO) * RSP;
    static_assert(PIECES % 64 == 0, "a buffer is filled by whole wave loads");
    constexpr int N_DMA = (PIECES + NT - 1) / NT;
    constexpr int MAIN_PIECES = VMHIP_TILE * RSP;

    extern __shared__ float4 lds4[];
    float* const w_lds = reinterpret_cast<float*>(lds4);
    float* const b_lds = w_lds + W_FLOATS;
    float* const buf0 = b_lds + 4;
    /* weights [slot][k / 4][output channel (4, zero padded)][k % 4]: lane (channel l % 4) reads four steps at once */
    for (int i = threadIdx.x; i < W_FLOATS; i += NT) {
        const int e = i % 4, o = (i / 4) % 4, k4 = (i / 16) % Q4, sl = i / (16 * Q4);
        w_lds[i] = o < C_OUT ? L.w[(size_t) (sl * C_IN + k4 * 4 + e) * C_OUT + o] : 0.0f;
    }
    if (threadIdx.x < 4) b_lds[threadIdx.x] = (int) threadIdx.x < C_OUT ? L.b[threadIdx.x] : 0.0f;

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int o_lane = lane & 3;
    const int activation = L.activation;

    const int n_tiles = vm_row_tiles(B);
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
    uint32_t hrow[N_DMA];
    auto request_halo_rows = [&](int t) {
#pragma unroll
        for (int k = 0; k < N_DMA; ++k) {
            const int p = threadIdx.x + k * NT;
            if ((k + 1) * NT > MAIN_PIECES) { /* compile-time: this k reaches into the halo rows */
                const int h = p / RSP - VMHIP_TILE;
                hrow[k] = __builtin_amdgcn_raw_buffer_load_b32(halo_rsrc, h >= 0 ? (t * VMHIP_HALO_MAX + h) * 4 : 0xffffffffu, 0, 0);
            }
        }
    };
    auto stage = [&](const int4& d, float* buf) {
#pragma unroll
        for (int k = 0; k < N_DMA; ++k) {
            if (k * NT + wave * 64 >= PIECES) continue; /* wave-uniform; only in a last, partial round */
            const int p = threadIdx.x + k * NT;
            const int row_l = p / RSP, cp = p - row_l * RSP;
            const int c = SWZ ? (cp ^ ((row_l >> 2) & 3)) : cp;
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
    };
    /* the lane's row of a tile: rows past the tile's count compute on its last row (the frame's null row) and skip
     * the store */
    auto own_row = [&](int rows_in_use) { return max(0, min((int) threadIdx.x, rows_in_use - 1)); };
    auto request_positions = [&](const int4& d) {
        return vm_load_nbl_row<NN>(nbl_rsrc, (d.x + own_row(d.y)) * (VMHIP_NBL_STRIDE * 2));
    };
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

    /* ---- prologue: the first tile (and, with two buffers, the second) on its way into LDS, the next ones described.
     * With two buffers the loop stages tile t+2 while t+1 waits in the other buffer; with one it stages t+1 into
     * the buffer tile t has just left and meets it again at the top of the loop. ---- */
    int t1 = tile + gx, t2 = tile + 2 * gx;
    int4 d_cur = load_desc(tile), d_n1 = load_desc(min(t1, t_last)), d_n2 = load_desc(min(t2, t_last));
    v4u nbl = {0, 0, 0, 0}, nbl_n1 = nbl, nbl_n2 = nbl;
    request_halo_rows(tile);
    stage(d_cur, buf0);
    nbl = request_positions(d_cur);
    if (NBUFS == 2 && t1 < t_end) {
        request_halo_rows(t1);
        stage(d_n1, buf0 + BUF_FLOATS);
        nbl_n1 = request_positions(d_n1);
    }
    request_halo_rows(min(NBUFS == 2 ? t2 : t1, t_last));
    d_cur = uniform(d_cur);
    if (NBUFS == 2) {
        wait_all_loads();
        __syncthreads(); /* weights, biases and the first tile are in LDS */
    }

    int cur = 0;
    while (true) {
        if (NBUFS == 1) {
            wait_all_loads();
            __syncthreads(); /* this tile (and, the first time, weights and biases) is in LDS */
        }
        const float* rows = buf0 + cur * BUF_FLOATS;
        const bool in_use = d_cur.y > 0;
        const bool valid = (int) threadIdx.x < d_cur.y;
        uint32_t li[SLOTS];
        bool far = false;
        li[0] = (uint32_t) own_row(d_cur.y);
#pragma unroll
        for (int s = 0; s < NN; ++s) {
            li[s + 1] = in_use ? nbl_entry(nbl, s) : 0u;
            far |= li[s + 1] >= FAR_FROM;
        }
        const bool any_far = __any(far);

        /* Two accumulators, even and odd input channels: a matrix instruction that adds to the result of the one right
         * before it waits for that result (the compiler puts two idle cycles between them); alternating, each finds its
         * operand ready. The first starts from the four channels' biases, the sum of the two is the row's result. */
        v4f accs[2] = {*reinterpret_cast<const v4f*>(b_lds), v4f{0.0f, 0.0f, 0.0f, 0.0f}};

        /* The operands come from LDS a quarter slot (four input channels) at a time: 16 bytes of the lane's source row and
         * 16 bytes of the slot's weights for its channel, four matrix instructions. A ring of Q4 quarters keeps the reads
         * one slot ahead of their use in half the registers of two whole slots. */
        auto contract = [&](auto far_tag) {
            constexpr bool FAR = decltype(far_tag)::value;
            if constexpr (!FAR) {
                constexpr int NQ = SLOTS * Q4, RING = Q4;
                float x[RING][4], a[RING][4];
                auto fetch = [&](int q, float (&xq)[4], float (&aq)[4]) {
                    const int sl = q / Q4, k4 = q % Q4;
                    const uint32_t at = li[sl];
                    load_floats<4>(rows + at * RS + ((SWZ ? (k4 ^ (int) ((at >> 2) & 3)) : k4) << 2), xq);
                    load_floats<4>(w_lds + ((sl * Q4 + k4) * 4 + o_lane) * 4, aq);
                };
#pragma unroll
                for (int r = 0; r < RING; ++r) fetch(r, x[r], a[r]);
#pragma unroll
                for (int q = 0; q < NQ; ++q) {
                    const int r = q % RING;
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int e = 0; e < 4; ++e) accs[e & 1] = __builtin_amdgcn_mfma_f32_4x4x1f32(a[r][e], x[r][e], accs[e & 1], 0, 0, 0);
                    if (q + RING < NQ) fetch(q + RING, x[r], a[r]);
                }
            }
            else {
                /* a tile with neighbours that are not staged: those lanes read their operands from global memory, slot by
                 * slot; same order of additions as above */
                float x[C_IN], a[C_IN];
#pragma unroll
                for (int sl = 0; sl < SLOTS; ++sl) {
                    const uint32_t at = li[sl] >= FAR_FROM ? 0u : li[sl];
#pragma unroll
                    for (int k4 = 0; k4 < Q4; ++k4) {
                        float t[4];
                        load_floats<4>(rows + at * RS + ((SWZ ? (k4 ^ (int) ((at >> 2) & 3)) : k4) << 2), t);
#pragma unroll
                        for (int e = 0; e < 4; ++e) x[k4 * 4 + e] = t[e];
                        load_floats<4>(w_lds + ((sl * Q4 + k4) * 4 + o_lane) * 4, t);
#pragma unroll
                        for (int e = 0; e < 4; ++e) a[k4 * 4 + e] = t[e];
                    }
                    if constexpr (NN > 0) {
                        if (sl > 0 && li[sl] >= FAR_FROM) {
                            const int g = B.row_nb[(size_t) (d_cur.x + li[0]) * B.nb_stride + (sl - 1)];
                            load_floats<C_IN>(in + (size_t) (d_cur.w + g) * C_IN, x);
                        }
                    }
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int k = 0; k < C_IN; ++k) accs[k & 1] = __builtin_amdgcn_mfma_f32_4x4x1f32(a[k], x[k], accs[k & 1], 0, 0, 0);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        };
        if (any_far) contract(std::true_type());
        else contract(std::false_type());
        v4f acc = accs[0] + accs[1];

        /* ---- every wave is done reading this buffer (with two buffers also: the next tile is complete and visible,
         * see conv_flow.hip) ---- */
        if (NBUFS == 2) wait_all_loads();
        __syncthreads();

        const bool has_next = t1 < t_end;
        const int t3 = t2 + gx;
        if (NBUFS == 2) {
            if (t2 < t_end) { /* uniform */
                stage(d_n2, buf0 + cur * BUF_FLOATS); /* tile t+2 into the buffer tile t just left */
                nbl_n2 = request_positions(d_n2);
            }
        }
        else if (has_next) {
            stage(d_n1, buf0); /* tile t+1 into the one buffer; the activation below overlaps its flight */
            nbl_n1 = request_positions(d_n1);
        }
        const int4 d_n3 = load_desc(min(t3, t_last));
        request_halo_rows(min(NBUFS == 2 ? t3 : t2, t_last));
        __builtin_amdgcn_sched_barrier(0);

        /* activation: the lane holds its row's channels 0..3. Softmax as the reference computes it (exp, then the division
         * by the row's sum, no shift by the maximum: apply_activation.hpp:57-64), with the hardware's exponential and
         * reciprocal: e^x = 2^(x log2 e) is off by at most |x| 1e-7 relative (the product's rounding) plus an ulp, the
         * reciprocal by an ulp - 3e-6 on a probability for logits up to 30, against a gate of 1e-4 - and the two take
         * a dozen instructions per row where the library's expf and an IEEE division take 150, which was a third of this
         * kernel's vector work per tile. */
        if (activation == VMHIP_SOFTMAX) {
            float sum = 0.0f;
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const float e = v < C_OUT ? __builtin_amdgcn_exp2f(acc[v] * 1.44269504088896340736f) : 0.0f;
                acc[v] = e;
                sum += e;
            }
            const float scale = __builtin_amdgcn_rcpf(sum);
#pragma unroll
            for (int v = 0; v < 4; ++v) acc[v] = acc[v] * scale;
        }
        else {
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const float t = acc[v];
                acc[v] = activation == VMHIP_SELU ? selu(t) : activation == VMHIP_RELU ? fmaxf(t, 0.0f) : tanhf(t);
            }
        }
        /* one row per lane, C_OUT consecutive floats; lanes without a row get an out-of-range offset */
        const __amdgpu_buffer_rsrc_t out_rsrc = make_rsrc(out + (size_t) d_cur.x * C_OUT, (uint64_t) VMHIP_TILE * C_OUT * 4);
        const uint32_t at = valid ? li[0] * C_OUT * 4 : 0xffffffffu;
        if constexpr (C_OUT == 4) {
            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4u, acc), out_rsrc, at, 0, 0);
        }
        else {
#pragma unroll
            for (int v = 0; v < C_OUT; ++v) __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(acc[v]), out_rsrc, valid ? at + v * 4 : 0xffffffffu, 0, 0);
        }

        if (!has_next) break;
        d_cur = uniform(d_n1);
        d_n1 = d_n2;
        d_n2 = d_n3;
        nbl = nbl_n1, nbl_n1 = nbl_n2;
        tile = t1;
        t1 = t2;
        t2 = t3;
        if (NBUFS == 2) cur ^= 1;
    }
    wait_all_loads(); /* no LDS load may outlive the wave */
}

template <int C_IN, int C_OUT, int SLOTS>
int launch_narrow(const VmBatchDev& B, const VmLayerDev& L, const float* in, float* out, hipStream_t stream) {
    constexpr size_t lds = narrow_lds_bytes(C_IN, SLOTS);
    static_assert(lds <= 160 * 1024, "weights and two row buffers must fit the CU's LDS");
    if ((uint64_t) B.n_row_tiles * VMHIP_TILE * C_IN * 4 > 0xffffffffull) return -1; /* 32-bit byte offsets */
    auto kernel = vm_conv_narrow_kernel<C_IN, C_OUT, SLOTS>;
    static std::atomic<bool> configured{false}; /* engines on several host threads may get here together */
    if (!configured) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, int(lds)) != hipSuccess) {
            (void) hipGetLastError();
            return -1;
        }
        configured = true;
    }
    int per_cu = int((160 * 1024) / (lds + 256));
    per_cu = per_cu < 1 ? 1 : per_cu > 4 ? 4 : per_cu;
    int grid = 256 * per_cu;
    const int need = ((B.n_row_tiles + 7) / 8) * 8;
    if (grid > need) grid = need;
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(NW * 64), lds, stream, B, L, in, out);
    return 0;
}

}  // namespace

#define VM_FOR_EACH_NARROW_SHAPE(X) \
    X(16, 3, 7)                     \
    X(16, 2, 7)                     \
    X(24, 4, 9)

bool vm_narrow_supported(int c_in, int c_out, int slots) {
#define X(CI, CO, SL) \
    if (c_in == CI && c_out == CO && slots == SL) return true;
    VM_FOR_EACH_NARROW_SHAPE(X)
#undef X
    return false;
}

int vm_launch_conv_narrow(const VmBatchDev& B, const VmLayerDev& L, const float* in, float* out, hipStream_t stream, const char** kernel_name) {
    if (B.n_row_tiles <= 0) return 0;
    if (!B.row_nbl || !B.tile_halo || !B.tile_desc || !L.w || L.in_bf16 || L.out_bf16 || L.arith_bf16) return -1;
#define X(CI, CO, SL)                                                       \
    if (L.c_in == CI && L.c_out == CO && L.slots == SL) {                   \
        if (kernel_name) *kernel_name = "conv_narrow_" #CI "x" #CO "s" #SL; \
        return launch_narrow<CI, CO, SL>(B, L, in, out, stream);            \
    }
    VM_FOR_EACH_NARROW_SHAPE(X)
#undef X
    return -1;
}

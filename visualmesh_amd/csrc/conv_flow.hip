/*
 * conv_flow.hip - the LDS-gather graph-convolution kernel without block-wide barriers in its tile loop: neighbour
 * gather + dense + bias + activation in one kernel (reference engine/cpu/engine.hpp:213-264,
 * apply_activation.hpp:34-84).
 *
 * Contraction, operand layout, tile-local tables, XCD-aware persistent tile walk and the side path for neighbours that
 * are not staged are those of conv_lds.hip; the rows go from global memory straight into LDS (buffer_load ... lds), into
 * two alternating row buffers. What differs most is how the 16 waves of a block stay in step. A barrier makes all of them change phase together, so
 * the matrix pipe idles whenever the block applies activations, stores or waits for the barrier itself. Here two
 * counters per row buffer, kept in LDS, take its place:
 *   staged[b]   += 1 by every loader once its share of a tile's loads has landed in buffer b,
 *   consumed[b] += 1 by every wave once it has read the last operand of the tile in buffer b.
 * A wave starts to contract tile k when staged[k & 1] says the tile is complete, and otherwise runs freely: while
 * one wave applies the activation and stores, the others on its SIMD keep the matrix pipe busy, and a wave that is
 * done early goes on with the next tile, which already lies in the other buffer.
 * The first four waves of the block (one per SIMD, and the ones the SIMDs serve first) are the loaders. Besides
 * contracting their rows like everyone else they bring in all data: a tile's rows, its rows of the neighbour table
 * and its descriptor go into the buffer; the descriptor and the halo row numbers of the tile after go into a slot
 * of the loader's own, from which it works out, right after a contraction, where each piece of that tile lies. It
 * issues those loads into buffer k & 1 once consumed[k & 1] says every wave is done with tile k; its loads of tile
 * k+1, issued a tile earlier, it reports right after its contraction of tile k.
 * Everything a wave waits for at step k depends only on what all waves do at step k-1, so the waits cannot form a
 * cycle; each is nevertheless bounded by a poll count, after which the wave tells its block, counts the event in
 * the batch's flow_timeouts word and leaves the tile loop, as does every wave that then sees the block's flag: no wave hangs and
 * none works on a tile that is not there. The host reads the count with every run and fails the run if it is not 0.
 * In the prologue loads are counted, not drained: a loader knows how many vector memory instructions it has issued
 * after the ones it needs (they complete in order) and waits with s_waitcnt vmcnt(that many), so the loads of the
 * second tile, in flight behind those of the first, are not waited for; every load is therefore issued
 * unconditionally, with an out-of-range offset where there is nothing to move. In the loop a loader waits once per
 * tile, right after its contraction, for everything it has in flight - all of it requested a contraction or more
 * ago. No load of the loop returns into a register: the compiler would wait for such a register by its own count,
 * which misses the loads written as assembly below, and a register carried round the loop while a load still fills
 * it forces a full drain at the copy.
 * A wave never ends with LDS loads in flight (the LDS could already belong to another block).
 */
#include <cstdlib>
#include <type_traits>

#include <atomic>

#include "vmhip_internal.h"

/* polls a wait may take (a poll is ~100 cycles, a tile ~20 000: the default is hundreds of tile periods, a fifth of a
 * second); only a test of the give-up path sets it, to something tiny (vmhip_debug_set) */
__device__ int vm_flow_poll_limit = VM_FLOW_POLL_LIMIT_DEFAULT;
hipError_t vm_flow_set_poll_limit(int polls) {
    return hipMemcpyToSymbol(HIP_SYMBOL(vm_flow_poll_limit), &polls, sizeof(polls));
}


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

constexpr int FLOW_WAVES = 16;
constexpr int FLOW_LOADERS = 4; /* measured: 8 loaders 2 % slower, every wave loading its own sixteenth 12 % slower */
/* wave priorities (s_setprio): contracting a tile while the tile before is still being read by others / contracting
 * the oldest unread tile / everything else. Measured on the 32 -> 32 layer: without the rule 152 us, with it 147 us;
 * "everything else" at 1 instead of 3: 158 us. */
#define FLOW_PRIO_AHEAD 0
#define FLOW_PRIO_BEHIND 2
#define FLOW_PRIO_REST 3
#define FLOW_SLEEP 1
constexpr int FLOW_HALO = 192; /* halo rows staged per tile: two tiles, their neighbour tables and the loaders' slots fit beside the weights */
/* rounds of NT loads that fill a buffer's rows, and how many of them reach into the halo rows */
__host__ __device__ constexpr int flow_rounds(int c_in) { return ((VMHIP_TILE + FLOW_HALO) * (row_stride(c_in) / 4) + FLOW_WAVES * 64 - 1) / (FLOW_WAVES * 64); }
__host__ __device__ constexpr int flow_halo_rounds(int c_in) { return flow_rounds(c_in) - VMHIP_TILE * (row_stride(c_in) / 4) / (FLOW_WAVES * 64); }
/* words of a loader's slot: a descriptor, then one halo row number per lane and load it will issue */
__host__ __device__ constexpr int flow_slot_words(int c_in) { return 4 + (FLOW_WAVES / FLOW_LOADERS) * flow_halo_rounds(c_in) * 64; }
__host__ __device__ constexpr size_t flow_lds_bytes(int c_in, int c_out, int slots) {
    return (size_t(slots) * (c_in / 4) * ((c_out + 15) / 16) * 64 + size_t((c_out + 15) / 16) * 16
            + 2 * (size_t(VMHIP_TILE + FLOW_HALO) * row_stride(c_in) + VMHIP_TILE * 4 + 4) + 8 + size_t(FLOW_LOADERS) * flow_slot_words(c_in)) * 4;
}

/* Polls an LDS counter until it has reached target (wrap-safe). False when the polls ran out or another wave of the
 * block has given up (the word after the four counters says so): the caller then leaves the tile loop without
 * touching the tile, whose descriptor and rows may not be there. The read is spelled out: a volatile access would
 * make the compiler wait for every vector memory instruction in flight as well. */
__device__ __forceinline__ bool wait_counter(const uint32_t* counter, const uint32_t* gave_up, uint32_t target, int polls) {
    const uint32_t at = (uint32_t) (uintptr_t) (const __attribute__((address_space(3))) uint32_t*) counter;
    const uint32_t flag_at = (uint32_t) (uintptr_t) (const __attribute__((address_space(3))) uint32_t*) gave_up;
    for (int spin = 0; spin < polls; ++spin) {
        uint32_t v, flag;
        asm volatile("ds_read_b32 %0, %2\n\tds_read_b32 %1, %3\n\ts_waitcnt lgkmcnt(0)" : "=&v"(v), "=&v"(flag) : "v"(at), "v"(flag_at) : "memory");
        if (__builtin_amdgcn_readfirstlane(flag) != 0) return false;
        if ((int32_t) (__builtin_amdgcn_readfirstlane(v) - target) >= 0) return true;
        __builtin_amdgcn_s_sleep(FLOW_SLEEP);
    }
    return false;
}

/* buffer_load ... lds spelled out: 16 (or 4) bytes per lane from a buffer offset straight into LDS at lds_base +
 * lane * 16 (or 4). Written as assembly so that the compiler does not know of it: it would otherwise make every
 * later LDS access, which it cannot tell apart from the load's target, wait for all such loads in flight - and the
 * whole point here is to read one buffer while the other fills. Ordering against the LDS reads is this file's
 * business (s_waitcnt vmcnt by count, and the counters). M0 is written without telling the compiler, which treats it
 * as reserved and sets it anew before each use of its own. */
__device__ __forceinline__ v4u raw_rsrc(const void* p, uint64_t bytes) {
    const uint64_t a = (uint64_t) p;
    return v4u{(uint32_t) a, (uint32_t) (a >> 32) & 0xffffu, bytes > 0xffffffffull ? 0xffffffffu : (uint32_t) bytes, 0x00020000u};
}
__device__ __forceinline__ uint32_t lds_address(const void* p) {
    return (uint32_t) (uintptr_t) (const __attribute__((address_space(3))) void*) p;
}
__device__ __forceinline__ void load_to_lds_b128(const v4u& rsrc, uint32_t lds_base, uint32_t offset) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds" ::"s"(lds_base), "v"(offset), "s"(rsrc) : "memory", "m0");
}
__device__ __forceinline__ void load_to_lds_b32(const v4u& rsrc, uint32_t lds_base, uint32_t offset) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dword %1, %2, 0 offen lds" ::"s"(lds_base), "v"(offset), "s"(rsrc) : "memory", "m0");
}

template <int C_IN, int C_OUT, int SLOTS>
__global__ __launch_bounds__(FLOW_WAVES * 64) void vm_conv_flow_kernel(VmBatchDev B, VmLayerDev L, const float* __restrict__ in, float* __restrict__ out) {
    constexpr int NW = FLOW_WAVES;
    constexpr int RB = VMHIP_TILE / (16 * NW);
    static_assert(NW * RB * 16 == VMHIP_TILE, "a block covers one tile");
    static_assert(C_IN % 4 == 0 && C_OUT % 4 == 0, "rows are staged and stored in 16-byte pieces");
    constexpr int NT = NW * 64;
    constexpr int STEPS = C_IN / 4;
    constexpr int CB = (C_OUT + 15) / 16;
    constexpr int NN = SLOTS - 1;
    static_assert(NN > 0 && NN <= VMHIP_NBL_STRIDE, "the tile-local neighbour table holds 8 entries per row");
    constexpr int RS = row_stride(C_IN);
    constexpr bool SWZ = row_swizzled(C_IN);
    constexpr uint32_t FAR_FROM = VMHIP_TILE + FLOW_HALO;
    constexpr int Q4 = C_IN / 4;  /* data pieces per row */
    constexpr int RSP = RS / 4;   /* pieces per LDS row, padding included */
    constexpr int W_FLOATS = SLOTS * STEPS * CB * 64;
    constexpr int G = STEPS % 4 == 0 ? 4 : STEPS % 2 == 0 ? 2 : 1; /* steps per LDS read */
    constexpr int CH = G;                                           /* steps per pipeline stage */
    constexpr int ROW_FLOATS = (VMHIP_TILE + FLOW_HALO) * RS;
    constexpr int NBL_AT = ROW_FLOATS;                 /* the tile's neighbour table (16 bytes per row) follows its rows */
    constexpr int DESC_AT = ROW_FLOATS + VMHIP_TILE * 4; /* and its descriptor follows that */
    constexpr int BUF_FLOATS = DESC_AT + 4;
    constexpr int PIECES = (VMHIP_TILE + FLOW_HALO) * RSP;
    static_assert(PIECES >= NT && NT * 4 == VMHIP_TILE * 16, "whole rounds of loads; the neighbour table is one round of 4 bytes per lane");
    constexpr int N_DMA = (PIECES + NT - 1) / NT; /* the last round overlaps the one before it instead of being partial */
    constexpr int MAIN_PIECES = VMHIP_TILE * RSP;
    constexpr int N_MAIN = MAIN_PIECES / NT;      /* rounds that fill nothing but the tile's own rows */
    constexpr int N_HALO = N_DMA - N_MAIN;        /* rounds that (also) fill halo rows: one row number each */
    /* The first LOADERS waves of the block - the oldest, which the SIMDs serve first, so they are done with a tile
     * long before the others - issue all loads, SHARE sixteenths of a tile each. Vector memory instructions of a
     * loader per tile: N_FILL for the tile itself (rows, neighbour table, descriptor), then N_AHEAD for what
     * staging the tile after needs (its descriptor into the loader's own slot, its halo row numbers). */
    constexpr int LOADERS = FLOW_LOADERS, SHARE = NW / LOADERS;
    constexpr int N_FILL = SHARE * (N_DMA + 1) + 1;
    constexpr int N_AHEAD = 1 + SHARE * N_HALO;
    static_assert(RB * CB + 2 * N_FILL + N_AHEAD < 64, "a loader's loads and stores in flight must fit the vmcnt counter");
    static_assert(N_DMA == flow_rounds(C_IN) && N_HALO == flow_halo_rounds(C_IN), "the LDS size is computed from the same rounds");
    constexpr int SLOT_WORDS = flow_slot_words(C_IN);

    extern __shared__ float4 lds4[];
    float* const w_lds = reinterpret_cast<float*>(lds4);
    float* const b_lds = w_lds + W_FLOATS;
    float* const buf0 = b_lds + CB * 16;
    uint32_t* const counters = reinterpret_cast<uint32_t*>(buf0 + 2 * BUF_FLOATS); /* staged[2], consumed[2] */
    if (threadIdx.x < 8) counters[threadIdx.x] = 0; /* staged[2], consumed[2], then the word that says a wave gave up */
    /* the weights lie in global memory in the order they have in LDS: whole waves of 16 bytes per lane, issued before
     * anything else so that they travel together with the first descriptors */
    static_assert(W_FLOATS % 256 == 0, "the weights are whole wave loads");
    {
        const v4u w_rsrc = raw_rsrc(L.w_flow, (uint64_t) W_FLOATS * 4);
        const int wave_at = __builtin_amdgcn_readfirstlane((int) (threadIdx.x >> 6));
        for (int i = wave_at * 256; i < W_FLOATS; i += NT * 4)
            load_to_lds_b128(w_rsrc, lds_address(w_lds + i), (uint32_t) (i + (threadIdx.x & 63) * 4) * 4u);
    }
    static_assert(CB * 16 <= NT, "one bias value per thread at most");
    const float my_bias = threadIdx.x < C_OUT ? L.b[threadIdx.x] : 0.0f; /* requested now, written to LDS before the barrier */

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int) (threadIdx.x >> 6));
    const int q = lane >> 4, r16 = lane & 15;
    const int activation = L.activation;
    const int lw = wave; /* which loader this wave is, if it is one */
    uint32_t* const slot = counters + 8 + SLOT_WORDS * (wave % LOADERS); /* a loader's notes on the tile it stages next */

    const int n_tiles = vm_row_tiles(B);
    const int xcd = blockIdx.x & 7, lb = blockIdx.x >> 3, gx = gridDim.x >> 3;
    const int per_xcd = (n_tiles + 7) >> 3;
    const int t_end = min(n_tiles, (xcd + 1) * per_xcd);
    const int tile0 = xcd * per_xcd + lb;
    if (tile0 >= t_end) return; /* the whole block leaves before any barrier or LDS load */
    const int t_last = t_end - 1;
    const int count = (t_end - tile0 + gx - 1) / gx; /* tiles of this block: tile0 + k * gx, k < count */

    const uint32_t total_rows = (uint32_t) n_tiles * VMHIP_TILE;
    auto make_rsrc = [](const void* p, uint64_t bytes) {
        return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, (int) (bytes > 0xffffffffull ? 0xffffffffu : (uint32_t) bytes), 0x00020000);
    };
    const v4u in_rsrc = raw_rsrc(in, (uint64_t) total_rows * C_IN * 4);
    const v4u nbl_rsrc = raw_rsrc(B.row_nbl, (uint64_t) total_rows * VMHIP_NBL_STRIDE * 2);
    const v4u desc_lds_rsrc = raw_rsrc(B.tile_desc, (uint64_t) n_tiles * 16);
    const __amdgpu_buffer_rsrc_t halo_rsrc = make_rsrc(B.tile_halo, (uint64_t) n_tiles * VMHIP_HALO_MAX * 4);
    const v4u halo_lds_rsrc = raw_rsrc(B.tile_halo, (uint64_t) n_tiles * VMHIP_HALO_MAX * 4);
    const __amdgpu_buffer_rsrc_t desc_rsrc = make_rsrc(B.tile_desc, (uint64_t) n_tiles * 16);

    /* Piece p of a buffer = 16 bytes at LDS row p / RSP, position p % RSP. Round r fills pieces first_piece(r) + t for
     * t = 0..NT-1; a loader plays threads (lw * SHARE + v) * 64 + lane, v < SHARE. */
    auto first_piece = [](int r) { return r * NT < PIECES - NT ? r * NT : PIECES - NT; };
    /* which halo row (of the tile's list) the lane's piece in halo round r of share v belongs to; negative: a main row */
    auto halo_index = [&](int v, int r) { return (first_piece(N_MAIN + r) + (lw * SHARE + v) * 64 + lane) / RSP - VMHIP_TILE; };
    /* the halo row numbers of tile t into registers (the prologue's way) */
    auto load_halo_rows = [&](int t, uint32_t (&hrow)[SHARE][N_HALO]) {
#pragma unroll
        for (int v = 0; v < SHARE; ++v)
#pragma unroll
            for (int r = 0; r < N_HALO; ++r) {
                const int h = halo_index(v, r);
                hrow[v][r] = __builtin_amdgcn_raw_buffer_load_b32(halo_rsrc, h >= 0 ? (t * VMHIP_HALO_MAX + h) * 4 : 0xffffffffu, 0, 0);
            }
    };
    /* descriptor and halo row numbers of tile t into the loader's slot (the loop's way: N_AHEAD loads) */
    auto request_ahead = [&](int t) {
        const uint32_t base = lds_address(slot);
        if (lane < 4) load_to_lds_b32(desc_lds_rsrc, base, t * 16 + lane * 4);
#pragma unroll
        for (int v = 0; v < SHARE; ++v)
#pragma unroll
            for (int r = 0; r < N_HALO; ++r) {
                const int h = halo_index(v, r);
                load_to_lds_b32(halo_lds_rsrc, base + (4 + (v * N_HALO + r) * 64) * 4, h >= 0 ? (uint32_t) ((t * VMHIP_HALO_MAX + h) * 4) : 0xffffffffu);
            }
    };
    /* where in the input each piece this loader fetches for a tile lies: first = the tile's first row, halo = its halo
     * rows, hrow(v, r) = the halo row number for the lane's piece; live = false moves nothing (zeros land in LDS) */
    auto plan = [&](int first, int halo, bool live, auto hrow, uint32_t (&offs)[SHARE][N_DMA]) {
#pragma unroll
        for (int v = 0; v < SHARE; ++v) {
            const int vt = (lw * SHARE + v) * 64 + lane;
#pragma unroll
            for (int r = 0; r < N_DMA; ++r) {
                const int p = first_piece(r) + vt;
                const int row_l = p / RSP, cp = p - row_l * RSP;
                const int c = SWZ ? (cp ^ (row_l & 7)) : cp;
                uint32_t off = (uint32_t) ((first + row_l) * Q4 + c) * 16u;
                if (r >= N_MAIN) {
                    const int h = row_l - VMHIP_TILE;
                    if (h >= 0) off = h < halo ? (hrow(v, r - N_MAIN) * Q4 + c) * 16u : 0xffffffffu;
                }
                if (RSP != Q4 && cp >= Q4) off = 0xffffffffu; /* padding piece */
                offs[v][r] = live ? off : 0xffffffffu;
            }
        }
    };
    /* the N_FILL loads of tile t */
    auto fill = [&](int t, int first, bool live, const uint32_t (&offs)[SHARE][N_DMA], float* buf) {
        const uint32_t base = lds_address(buf);
#pragma unroll
        for (int v = 0; v < SHARE; ++v) {
#pragma unroll
            for (int r = 0; r < N_DMA; ++r) load_to_lds_b128(in_rsrc, base + (first_piece(r) + (lw * SHARE + v) * 64) * 16, offs[v][r]);
            /* the tile's rows of the neighbour table, 4 bytes per lane */
            load_to_lds_b32(nbl_rsrc, base + (NBL_AT + (lw * SHARE + v) * 64) * 4,
                            live ? (uint32_t) (first * (VMHIP_NBL_STRIDE * 2) + ((lw * SHARE + v) * 64 + lane) * 4) : 0xffffffffu);
        }
        /* and its descriptor (every loader writes the same four words) */
        if (lane < 4) load_to_lds_b32(desc_lds_rsrc, base + DESC_AT * 4, live ? (uint32_t) (t * 16 + lane * 4) : 0xffffffffu);
    };
    auto own_row = [&](int rows_in_use, int rb) { return max(0, min(wave * (RB * 16) + rb * 16 + r16, rows_in_use - 1)); };
    /* Descriptors travel through vector memory (a scalar load in flight would turn every LDS wait into a full
     * wait). Inside the loop they go into an LDS slot of the wave's own, not into registers: a register that is
     * the target of a load in flight cannot be carried round the loop without waiting for that load, and for all
     * loads before it, at the copy. */
    auto load_desc = [&](int t) {
        const v4u d = __builtin_amdgcn_raw_buffer_load_b128(desc_rsrc, t * 16, 0, 0);
        return make_int4(__builtin_amdgcn_readfirstlane((int) d.x), __builtin_amdgcn_readfirstlane((int) d.y),
                         __builtin_amdgcn_readfirstlane((int) d.z), __builtin_amdgcn_readfirstlane((int) d.w));
    };
    auto read_desc = [&](const void* at) {
        const v4u d = *reinterpret_cast<const v4u*>(at);
        return make_int4(__builtin_amdgcn_readfirstlane((int) d.x), __builtin_amdgcn_readfirstlane((int) d.y),
                         __builtin_amdgcn_readfirstlane((int) d.z), __builtin_amdgcn_readfirstlane((int) d.w));
    };
    auto tile_of = [&](int k) { return min(tile0 + k * gx, t_last); };
    const int polls = vm_flow_poll_limit;
    uint32_t* const gave_up = counters + 4;
    /* a wait ran out: tell the block, count it for the host, and (the caller) leave the loop */
    auto give_up = [&] {
        if (lane == 0) {
            atomicOr(gave_up, 1u);
            atomicAdd(B.flow_timeouts, 1u);
        }
    };

    /* ---- prologue: tiles 0 and 1 on their way into the two buffers, tile 2 described ---- */
    const bool loader = lw < LOADERS;
    uint32_t offs[SHARE][N_DMA]; /* a loader's plan for the tile it fills next */
    int first_new = 0;
    if (loader) {
        uint32_t h0[SHARE][N_HALO], h1[SHARE][N_HALO];
        load_halo_rows(tile_of(0), h0);
        load_halo_rows(tile_of(1), h1);
        const int4 d0 = load_desc(tile_of(0)), d1 = load_desc(tile_of(1));
        /* Name every register a load fills before the first load that the compiler does not know of: it waits for
         * such a register by counting the vector memory instructions it knows were issued after the load, so a
         * wait placed later would drain the unknown ones too. */
#pragma unroll
        for (int v = 0; v < SHARE; ++v)
#pragma unroll
            for (int r = 0; r < N_HALO; ++r) asm volatile("" ::"v"(h0[v][r]), "v"(h1[v][r]));
        if (threadIdx.x < CB * 16) b_lds[threadIdx.x] = my_bias;
        request_ahead(tile_of(2));
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N_AHEAD) : "memory"); /* my part of the weights (requested first of all) */
        __syncthreads(); /* weights, biases and the zeroed counters are in LDS */
        plan(d0.x, d0.z, true, [&](int v, int r) { return h0[v][r]; }, offs);
        fill(tile_of(0), d0.x, true, offs, buf0);
        plan(d1.x, d1.z, 1 < count, [&](int v, int r) { return h1[v][r]; }, offs);
        fill(tile_of(1), d1.x, 1 < count, offs, buf0 + BUF_FLOATS);
        /* tile 0 has landed once only the loads of tile 1 can still be in flight */
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N_FILL) : "memory");
        if (lane == 0) atomicAdd(&counters[0], 1u);
    }
    else {
        if (threadIdx.x < CB * 16) b_lds[threadIdx.x] = my_bias;
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); /* my part of the weights */
        __syncthreads();
    }

    for (int k = 0; k < count; ++k) {
        const int b = k & 1;
        const uint32_t round = (uint32_t) ((k >> 1) + 1); /* the round of buffer b that tile k is */
        const float* rows = buf0 + b * BUF_FLOATS;

        if (!wait_counter(&counters[b], gave_up, LOADERS * round, polls)) { /* every loader's share of tile k has landed */
            give_up();
            break;
        }
        const int4 d_cur = read_desc(rows + DESC_AT);
        /* The SIMDs serve their oldest wave first, so left alone the youngest falls a whole tile behind, and the
         * buffer it still reads cannot be refilled. A wave that starts a tile while the tile before is not yet
         * read by all therefore steps back behind those that are still on it. */
        {
            uint32_t before = 0;
            if (k > 0) {
                const uint32_t at = lds_address(&counters[2 + (b ^ 1)]);
                asm volatile("ds_read_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(before) : "v"(at) : "memory");
                before = __builtin_amdgcn_readfirstlane(before);
            }
            if (k == 0 || (int32_t) (before - NW * (uint32_t) (((k - 1) >> 1) + 1)) >= 0) __builtin_amdgcn_s_setprio(FLOW_PRIO_BEHIND);
            else __builtin_amdgcn_s_setprio(FLOW_PRIO_AHEAD);
        }

        const bool in_use = d_cur.y > 0;
        v4u nbl[RB];
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) nbl[rb] = *reinterpret_cast<const v4u*>(rows + NBL_AT + own_row(d_cur.y, rb) * 4);
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
                if constexpr (FAR) {
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
                const int s = FAR ? 0 : (c & 1);
                if constexpr (FAR) {
                    gather(c, x[0]);
                    weights(c, a[0]);
                }
                else if (c + 1 < CHUNKS) {
                    gather(c + 1, x[s ^ 1]);
                    weights(c + 1, a[s ^ 1]);
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int e = 0; e < CH; ++e)
#pragma unroll
                    for (int cb = 0; cb < CB; ++cb)
#pragma unroll
                        for (int rb = 0; rb < RB; ++rb)
                            acc[rb][cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[s][cb][e], x[s][rb][e], acc[rb][cb], 0, 0, 0);
                if constexpr (FAR) __builtin_amdgcn_sched_barrier(0);
            }
        };
        if (any_far) {
            contract(std::true_type());
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); /* the side path's loads: none may be counted below */
        }
        else {
            contract(std::false_type());
        }
        /* every operand of the tile has been read (the matrix instructions above consumed them) */
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        if (lane == 0) atomicAdd(&counters[2 + b], 1u);
        __builtin_amdgcn_s_setprio(FLOW_PRIO_REST); /* what follows is short and keeps no matrix pipe busy: let it through */
        if (loader) {
            /* The notes on tile k+2, requested a tile ago, are in the slot once nothing but what was requested after
             * them can still be in flight: the loads of tile k+1 and the stores of tile k-1 (of tiles 0 and 1 at first). */
            /* Everything in flight was requested at least a contraction ago - the notes on tile k+2, the stores of
             * tile k-1, my share of tile k+1 - so it has landed or is about to: tile k+1 is reported here, before the
             * activation, and a wave that is done with tile k early can go on (reporting it only after the stores,
             * with a wait by count that let them stay in flight, was 3 % slower on the 32 -> 32 layer). */
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            if (lane == 0) atomicAdd(&counters[b ^ 1], 1u);
            const int4 d_new = read_desc(slot);
            first_new = d_new.x;
            plan(d_new.x, d_new.z, k + 2 < count, [&](int v, int r) { return slot[4 + (v * N_HALO + r) * 64 + lane]; }, offs);
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); /* the slot has been read: it may be written again */
            request_ahead(tile_of(k + 3));
        }

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
                __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4u, acc[rb][cb]), out_rsrc, (valid[rb] && o < C_OUT) ? at : 0xffffffffu, 0, 0);
            }
        }

        if (loader) {
            /* my share of tile k+1, requested a tile ago, has landed once nothing but what was requested after it and
             * the stores above can still be in flight */
            /* tile k+2 goes where tile k was, once every wave has read the last of tile k */
            if (!wait_counter(&counters[2 + b], gave_up, NW * round, polls)) {
                give_up();
                break;
            }
            fill(tile_of(k + 2), first_new, k + 2 < count, offs, buf0 + b * BUF_FLOATS);
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); /* no LDS load may outlive the wave */
}

template <int C_IN, int C_OUT, int SLOTS>
int launch_flow(const VmBatchDev& B, const VmLayerDev& L, const float* in, float* out, hipStream_t stream) {
    constexpr size_t lds = flow_lds_bytes(C_IN, C_OUT, SLOTS);
    static_assert(lds <= 160 * 1024, "weights, two row buffers and the counters must fit the CU's LDS");
    /* the kernel addresses its input rows with 32-bit byte offsets */
    if ((uint64_t) B.n_row_tiles * VMHIP_TILE * C_IN * 4 > 0xffffffffull) return -1;
    auto kernel = vm_conv_flow_kernel<C_IN, C_OUT, SLOTS>;
    static std::atomic<bool> configured{false}; /* engines on several host threads may get here together */
    if (!configured) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, int(lds)) != hipSuccess) {
            (void) hipGetLastError();
            return -1;
        }
        configured = true;
    }
    int grid = 256; /* one block of 16 waves per CU */
    const int need = ((B.n_row_tiles + 7) / 8) * 8;
    if (grid > need) grid = need;
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(FLOW_WAVES * 64), lds, stream, B, L, in, out);
    return 0;
}

}  // namespace

#define VM_FOR_EACH_FLOW_SHAPE(X) \
    X(16, 16, 7)                  \
    X(16, 32, 7)                  \
    X(32, 32, 7)                  \
    X(32, 16, 7)

void vm_flow_order_weights(const float* w_mfma, int c_in, int c_out, int slots, float* out) {
    const int STEPS = c_in / 4, CB = (c_out + 15) / 16;
    const int G = STEPS % 4 == 0 ? 4 : STEPS % 2 == 0 ? 2 : 1;
    const int n = slots * STEPS * CB * 64;
    for (int i = 0; i < n; ++i) {
        const int e = i % G, l = (i / G) % 64, jg = (i / (G * 64)) % (STEPS / G), cb = (i / (G * 64 * (STEPS / G))) % CB, sl = i / (STEPS * 64 * CB);
        out[i] = w_mfma[((sl * STEPS + jg * G + e) * CB + cb) * 64 + l];
    }
}

bool vm_flow_supported(int c_in, int c_out, int slots) {
#define X(CI, CO, SL) \
    if (c_in == CI && c_out == CO && slots == SL) return true;
    VM_FOR_EACH_FLOW_SHAPE(X)
#undef X
    return false;
}

int vm_launch_conv_flow(const VmBatchDev& B, const VmLayerDev& L, const float* in, float* out, hipStream_t stream, const char** kernel_name) {
    if (B.n_row_tiles <= 0) return 0;
    if (!B.row_nbl || !B.tile_halo || !B.tile_desc || !L.w_flow || L.in_bf16 || L.out_bf16 || L.arith_bf16) return -1;
#define X(CI, CO, SL)                                                     \
    if (L.c_in == CI && L.c_out == CO && L.slots == SL) {                 \
        if (kernel_name) *kernel_name = "conv_flow_" #CI "x" #CO "s" #SL; \
        return launch_flow<CI, CO, SL>(B, L, in, out, stream);            \
    }
    VM_FOR_EACH_FLOW_SHAPE(X)
#undef X
    return -1;
}

/*
 * conv_bf16.hip - graph-convolution layers of the bf16 engine (64 -> 64 channels) on the bf16 matrix instructions of
 * gfx950 with fp32 accumulation: neighbour gather + dense + bias + activation in one kernel (reference
 * engine/cpu/engine.hpp:213-264, apply_activation.hpp:34-84).
 *
 * Instruction: v_mfma_f32_32x32x16_bf16, a 32 (output channels) x 32 (rows) block over 16 values of the reduction
 * index; it runs at twice the rate of the 16x16x32 form on this hardware.
 *   A operand: lane l supplies W[k(l / 32, e)][o = l % 32], e = 0..7     (weights)
 *   B operand: lane l supplies in[src(row = l % 32)][k(l / 32, e)]        (gathered rows)
 *   D:         lane l holds, for row l % 32, channels 8 * g + 4 * (l / 32) + {0..3}, g = 0..3
 * The reduction index may be permuted freely as long as both operands agree: in step j of a gather slot lane half
 * h = l / 32 takes the 16-byte piece 4 * h + j of the gathered row (eight consecutive channels).
 *
 * Where things live. The weights of a layer, 7 x 64 x 64 values as hi + lo pairs of bf16 (114 KB), stay in REGISTERS
 * for the life of a persistent block of four waves, one wave per SIMD with all 512 registers of a lane: wave w holds
 * the 32 output channels of channel block w % 2 (224 registers per lane) and works on the 64 rows of row half w / 2.
 * That leaves the whole LDS to the rows: a half tile (VMHIP_HTILE = 128 rows) and the rows of other half tiles that
 * its neighbour table names (its halo, up to VMHIP_HHALO = 128) are brought in once per half tile by
 * buffer_load ... lds, whole cache lines per request, into one of two alternating buffers, and the B operands are
 * gathered from there with ds_read_b128. (With the weights in LDS there is no room for rows, every gathered row is
 * then fetched seven times by lanes that each touch another cache line, and the kernel is bound by the vector cache:
 * 8.3 ms per launch.) 16-byte pieces are XOR-swizzled with the row's number so that sixteen lanes reading the same
 * piece of sixteen consecutive rows - what the LDS serves per cycle - meet no bank twice.
 *
 * Precision. Weights are w = hi + lo with hi = bf16(w), lo = bf16(w - hi): they cost no accuracy. Rows come in three
 * formats (VM_ROWS_*): bf16 (the one rounding the bf16 engine allows itself at some layer boundaries), hi + lo pairs of
 * bf16 (the size of an fp32 row, split once by the layer that produces the row) or fp32 (split in registers at every
 * use; only for a bf16 layer behind a kernel that cannot write the split form). A layer reading bf16 rows issues
 * x*w_hi + x*w_lo per step, the others x_hi*w_hi + x_lo*w_hi + x_hi*w_lo (what is dropped, x_lo*w_lo, is 2^-17 of a
 * product).
 *
 * Schedule of a block. Per half tile k: wait until my own loads of it have landed (they were issued a half tile
 * ago; s_waitcnt vmcnt by count, so that the stores issued since stay in flight), one barrier (everyone's have
 * landed, and everyone is done reading the other buffer), issue the loads of half tile k+1 into the other buffer
 * from the note (descriptor + halo rows) that was requested a half tile ago, request the note of k+2, then the matrix
 * work of k - into which the activation and stores of half tile k-1, whose accumulators are kept, are scheduled by
 * the compiler: a matrix instruction occupies the pipe for 32 cycles and takes 4 to issue, the rest belongs to the
 * vector ALU. Every load and store is issued unconditionally (out-of-range offsets move nothing) so that the counts
 * are constants.
 */
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <type_traits>
#include <utility>

#include <atomic>

#include "vmhip_internal.h"


/* The activation code of this file is compiled three times per kernel (the usual half tile, the one with neighbours that
 * are not staged, the last half tile of a block): no contraction of a multiplication and an addition at the compiler's
 * discretion, which may differ between the copies - a row's result must not depend on which copy computed it. Where a
 * fused multiply-add is wanted it is written out. */
#pragma clang fp contract(off)

namespace {

typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef uint32_t v4u __attribute__((ext_vector_type(4)));
typedef uint32_t v2u __attribute__((ext_vector_type(2)));

constexpr int BT = VMHIP_HTILE;   /* rows of a half tile */
constexpr int BH = VMHIP_HHALO;   /* halo rows staged beside them */
constexpr int BROWS = BT + BH;    /* LDS rows per buffer */
constexpr int NOTE = VMHIP_NOTE_WORDS;
constexpr int CH = 64;            /* channels in and out */
constexpr uint32_t OOR = 0xffffffffu; /* a buffer offset that is out of range: the load returns zeros, the store is dropped */

__device__ __forceinline__ int find_frame_by_row_tile(const VmFrame* frames, int n, int tile) {
    int lo = 0, hi = n - 1;
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (frames[mid].row_tile0 <= tile) lo = mid;
        else hi = mid - 1;
    }
    return lo;
}

/* body(integral_constant<int, 0>) ... body(integral_constant<int, N - 1>): a loop whose index is a constant in every
 * round, whatever the optimiser thinks of the size of what it unrolls (an index that stayed a variable would put the
 * weights, an array in registers, into scratch memory) */
template <class F, int... I>
__device__ __forceinline__ void static_for_impl(F&& body, std::integer_sequence<int, I...>) {
    (body(std::integral_constant<int, I>()), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F&& body) {
    static_for_impl(body, std::make_integer_sequence<int, N>());
}

/* selu with the hardware exponential: the branch that needs it has s < 0, where alpha * e^s - alpha is off by at most
 * ~3e-7 absolute against the correctly rounded result */
__device__ __forceinline__ float selu(float s) {
    const float lambda = 1.0507009873554804934193349852946f;
    const float alpha = 1.6732632423543772848170429916717f;
    return lambda * (s >= 0.0f ? s : __builtin_fmaf(alpha, __builtin_amdgcn_exp2f(s * 1.44269504088896340736f), -alpha));
}

/* tanh(x) = 1 - 2 / (e^(2x) + 1) with the hardware exponential and reciprocal: within ~3e-7 absolute of the correctly
 * rounded result over the whole range (e^(2x) overflows to infinity and underflows to zero where tanh is +-1), in a
 * handful of instructions and two registers - the library routine's polynomial needs enough of both to push the kernel's
 * working set out of the register file */
__device__ __forceinline__ float fast_tanh(float x) {
    const float t = __builtin_amdgcn_exp2f(x * 2.88539008177792681472f); /* 2 log2 e */
    return __builtin_fmaf(-2.0f, __builtin_amdgcn_rcpf(t + 1.0f), 1.0f);
}

/* two floats -> two bf16 in one word, round to nearest even (v_cvt_pk_bf16_f32) */
__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
    typedef __bf16 v2bf __attribute__((ext_vector_type(2)));
    v2bf t;
    t[0] = (__bf16) a;
    t[1] = (__bf16) b;
    return __builtin_bit_cast(uint32_t, t);
}
__device__ __forceinline__ float bf16_low(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf16_high(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }
/* hi and lo words of a pair of floats: hi = bf16(x), lo = bf16(x - hi); the difference is exact in fp32 */
__device__ __forceinline__ void split_pair(float a, float b, uint32_t& hi, uint32_t& lo) {
    hi = pack_bf16(a, b);
    lo = pack_bf16(a - bf16_low(hi), b - bf16_high(hi));
}
/* eight floats (two 16-byte pieces) -> eight hi and eight lo bf16 */
__device__ __forceinline__ void split_eight(const v4u& f0, const v4u& f1, v4u& hi, v4u& lo) {
    uint32_t h0, h1, h2, h3, l0, l1, l2, l3;
    split_pair(__uint_as_float(f0.x), __uint_as_float(f0.y), h0, l0);
    split_pair(__uint_as_float(f0.z), __uint_as_float(f0.w), h1, l1);
    split_pair(__uint_as_float(f1.x), __uint_as_float(f1.y), h2, l2);
    split_pair(__uint_as_float(f1.z), __uint_as_float(f1.w), h3, l3);
    hi = v4u{h0, h1, h2, h3};
    lo = v4u{l0, l1, l2, l3};
}

/* the k-th 16-bit entry of a row of the half-tile neighbour table */
__device__ __forceinline__ uint32_t nbl_entry(const v4u& t, int k) {
    const uint32_t w = (k >> 1) == 0 ? t.x : (k >> 1) == 1 ? t.y : (k >> 1) == 2 ? t.z : t.w;
    return (k & 1) ? (w >> 16) : (w & 0xffffu);
}

/* buffer_load ... lds spelled out: 16 (or 4) bytes per lane from a buffer offset straight into LDS at lds_base +
 * lane * 16 (or 4). Written as assembly so that the compiler does not know of it: it would otherwise make every
 * later LDS access, which it cannot tell apart from the load's target, wait for all such loads in flight - and the
 * whole point here is to read one buffer while the other fills. Ordering against the LDS reads is this file's
 * business (s_waitcnt vmcnt by count, and the barrier). */
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

__host__ __device__ constexpr int row_bytes(int fmt) { return fmt == VM_ROWS_BF16 ? CH * 2 : CH * 4; }
__host__ __device__ constexpr int bf16_buf_bytes(int in_fmt) { return BROWS * row_bytes(in_fmt) + BT * 16; }
/* two row buffers (rows, then the half tile's neighbour table), a note per wave, the biases, the softmax's exchange */
__host__ __device__ constexpr size_t bf16_lds_bytes(int in_fmt) { return 2 * size_t(bf16_buf_bytes(in_fmt)) + 4 * NOTE * 4 + CH * 4 + BT * 2 * 4; }

/* the side work of a half tile in the order it is issued: every FILL_EVERY-th item is a load of the half tile after, the
 * others are the pieces of the half tile before */
constexpr int FILL_EVERY = 3;
constexpr int slice_of_item(int item, int n_fill) { return item - (item / FILL_EVERY + 1 < n_fill ? item / FILL_EVERY + 1 : n_fill); }
/* stores (pieces 32.., of which with fp32 or bf16 rows out only the even ones store) issued after the last load */
/* whether piece sl of a half tile's results stores: pieces 32 + 2 u and 33 + 2 u belong to unit u = (row block, g). fp32
 * rows out: the first piece of every unit (four channels, 16 bytes); bf16 rows out: the first piece of the units with even
 * g (eight channels, 16 bytes); hi + lo rows out: both pieces of those units (the hi parts, then the lo parts) */
constexpr bool slice_stores(int sl, int out_fmt) {
    if (sl < 32) return false;
    const int g = ((sl - 32) >> 1) & 3, part = (sl - 32) & 1;
    return out_fmt == VM_ROWS_F32 ? part == 0 : out_fmt == VM_ROWS_BF16 ? (g % 2 == 0 && part == 0) : g % 2 == 0;
}
constexpr int stores_after_fills(int n_fill, int n_slices, int out_fmt) {
    int n = 0;
    for (int item = FILL_EVERY * (n_fill - 1) + 1; slice_of_item(item, n_fill) < n_slices; ++item)
        if (slice_stores(slice_of_item(item, n_fill), out_fmt)) ++n;
    return n;
}

/* what a wave remembers of a half tile until its results are stored */
struct Done {
    uint32_t first; /* the half tile's first row in the batch */
    uint32_t own[2]; /* the lane's row of each row block within the half tile */
    bool valid[2];   /* ... and whether that row is in use */
};

template <int SLOTS, int IN_FMT, int OUT_FMT, int ACT>
__global__ __launch_bounds__(256) void vm_conv_bf16_kernel(VmBatchDev B, VmLayerDev L, const void* __restrict__ in, void* __restrict__ out) {
    constexpr int NN = SLOTS - 1;
    static_assert(NN > 0 && NN <= VMHIP_NBL_STRIDE, "the half-tile neighbour table holds 8 entries per row");
    constexpr int ROWB = row_bytes(IN_FMT);   /* bytes of an input row */
    constexpr int OUTB = row_bytes(OUT_FMT);
    /* A buffer holds the rows as planes of 128-byte half rows (bf16 rows: one plane; hi + lo rows: the hi plane, then
     * the lo plane; fp32 rows: channels 0..31, then channels 32..63), so that a lane finds the lo part of an operand at
     * a constant distance from the hi part, and so that the bank a 16-byte piece lies in depends on four bits of
     * (row, piece): what the LDS serves per cycle is sixteen lanes' pieces if they lie in sixteen different quarters of
     * a 256-byte bank line. Piece q of half row R lies at R * 128 + (q ^ ((R >> 1) & 7)) * 16. */
    constexpr int PLANES = ROWB / 128;
    constexpr int PLANE = BROWS * 128;        /* bytes of a plane */
    constexpr int RPR = 32;                   /* half rows filled per round of 256 lanes */
    constexpr int NRP = BROWS / RPR;          /* rounds per plane */
    constexpr int NRP_OWN = BT / RPR;         /* ... of which these fill the half tile's own rows */
    constexpr int NR = NRP * PLANES;          /* rounds per buffer */
    constexpr int BUF = bf16_buf_bytes(IN_FMT);
    constexpr int NBL_AT = BROWS * ROWB;      /* the half tile's neighbour table follows its rows */
    constexpr bool WIDE = IN_FMT != VM_ROWS_BF16; /* inputs come as hi + lo */
    constexpr int N_STORES = OUT_FMT == VM_ROWS_BF16 ? 4 : 8; /* vector stores of a wave per half tile */
    constexpr int N_FILL = NR + 2;            /* loads of a wave per half tile: rows, neighbour table */
    static_assert(N_STORES + N_FILL + 3 < 64, "what a wave has in flight must fit the vmcnt counter");

    extern __shared__ float4 lds4[];
    char* const lds = reinterpret_cast<char*>(lds4);
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int) (threadIdx.x >> 6));
    const int cb = wave & 1, rh = wave >> 1;
    const int h = lane >> 5, r32 = lane & 31;
    uint32_t* const slot = reinterpret_cast<uint32_t*>(lds + 2 * BUF) + wave * NOTE;
    float* const b_lds = reinterpret_cast<float*>(lds + 2 * BUF + 4 * NOTE * 4);
    float* const xch = b_lds + CH;

    /* half tiles in use, and this block's share: XCD-aware (block b works for XCD b % 8 on a contiguous eighth) */
    const int n_tiles = B.active_h[B.n_frames];
    const int xcd = blockIdx.x & 7, lb = blockIdx.x >> 3, gx = gridDim.x >> 3;
    const int per_xcd = (n_tiles + 7) >> 3;
    const int t_end = min(n_tiles, (xcd + 1) * per_xcd);
    const int tile0 = xcd * per_xcd + lb;
    if (tile0 >= t_end) return; /* the whole block leaves before any barrier or LDS load */
    const int count = (t_end - tile0 + gx - 1) / gx; /* half tiles of this block: tile0 + k * gx, k < count */

    /* the wave's weights: [channel block][slot][step][hi, lo][lane] 16 bytes each */
    v4u w[SLOTS][4][2];
    {
        const v4u* wp = reinterpret_cast<const v4u*>(L.w_mfma) + (size_t) cb * (SLOTS * 4 * 2 * 64) + lane;
#pragma unroll
        for (int s = 0; s < SLOTS; ++s)
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int p = 0; p < 2; ++p) w[s][j][p] = wp[((s * 4 + j) * 2 + p) * 64];
    }
    if (threadIdx.x < CH) b_lds[threadIdx.x] = L.b[threadIdx.x];
    /* Every load the compiler knows of returns before the first one it does not know of is issued. The same statements
     * say where the weights live: in accumulation registers ("a"), from which the matrix instruction reads them as well
     * as from vector registers. Left to itself the compiler keeps the 224 weight registers in the vector file and moves
     * everything else in and out of accumulation registers around each use (822 such moves in the kernel against 176, a
     * sixth of its instructions; 4-5 % of its time).
     * No instantiation may spill to scratch memory. With the weights placed like this the compiler (ROCm 7.2's clang)
     * spills a weight's four registers as three words to scratch plus one word kept in a spare vector register, and at
     * the use reloads the three words only (scratch_load_dwordx3 v[24:26], then v_mfma ... v[24:27]): the matrix
     * instruction multiplies with whatever the fourth register last held, and the results are garbage, NaNs included.
     * That is what instantiations with a library tanh did (its polynomial's registers pushed 18 to 30 values out); with
     * fast_tanh above they all fit. The two that still do not (fp32 rows in, hi + lo rows out, selu or tanh: the splitting of
     * rows in registers on top of the widest epilogue) keep the weights where the compiler puts them, and fit that way.
     * tests/test_abi.py compiles this file and checks that none of the 36 kernels has a scratch segment. */
    constexpr bool WEIGHTS_IN_AGPRS = !(IN_FMT == VM_ROWS_F32 && OUT_FMT == VM_ROWS_BF16X2 && (ACT == VMHIP_SELU || ACT == VMHIP_TANH));
#pragma unroll
    for (int s = 0; s < SLOTS; ++s)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int p = 0; p < 2; ++p) {
                if constexpr (WEIGHTS_IN_AGPRS) asm volatile("" : "+a"(w[s][j][p]));
                else asm volatile("" : "+v"(w[s][j][p]));
            }

    const uint32_t total_rows = (uint32_t) B.n_row_tiles * VMHIP_TILE;
    const v4u note_rsrc = raw_rsrc(B.tile_note_h, (uint64_t) n_tiles * NOTE * 4);
    const v4u nbl_rsrc = raw_rsrc(B.row_nbl_h, (uint64_t) total_rows * VMHIP_NBL_STRIDE * 2);

    /* the note of half tile t into the wave's slot: 3 loads */
    auto request_note = [&](int t, bool live) {
        const uint32_t base = lds_address(slot);
        const uint32_t off = live ? (uint32_t) (t * NOTE + lane) * 4u : OOR;
        load_to_lds_b32(note_rsrc, base, off);
        load_to_lds_b32(note_rsrc, base + 256, live ? off + 256 : OOR);
        if (lane < NOTE - 128) load_to_lds_b32(note_rsrc, base + 512, live ? off + 512 : OOR);
    };
    auto read_note = [&]() {
        const v4u d = *reinterpret_cast<const v4u*>(slot);
        return make_int4(__builtin_amdgcn_readfirstlane((int) d.x), __builtin_amdgcn_readfirstlane((int) d.y),
                         __builtin_amdgcn_readfirstlane((int) d.z), __builtin_amdgcn_readfirstlane((int) d.w));
    };
    /* Round r = plane * NRP + i fills half rows 32 i .. 32 i + 31 of that plane: thread t brings the 16 bytes at
     * position t % 8 of half row 32 i + t / 8, which are piece (t % 8) ^ swizzle of that half of the source row. The
     * swizzle only depends on the thread, not on the round. */
    const int my_row = (int) threadIdx.x / 8, my_cp = (int) threadIdx.x % 8;
    const int my_sw = (my_row >> 1) & 7;
    const uint32_t my_piece = (uint32_t) ((my_cp ^ my_sw) * 16);
    /* The N_FILL loads of a half tile, one at a time (fill_item), after its note has been read from the slot
     * (plan_fill: the descriptor, and the halo row each of this thread's pieces of a halo round belongs to). */
    struct Plan {
        v4u in_rsrc;
        uint32_t base, own0, nbl0;
        uint32_t halo_off[NRP - NRP_OWN];
    };
    auto plan_fill = [&](const int4& d, bool live, int b, Plan& P) {
        /* offsets are relative to the frame's first row: a frame's rows fit 32 bits, a batch's need not */
        const uint32_t rows_left = total_rows - (uint32_t) d.w;
        P.in_rsrc = raw_rsrc(reinterpret_cast<const char*>(in) + (size_t) (uint32_t) d.w * ROWB, (uint64_t) rows_left * ROWB);
        P.base = lds_address(lds + b * BUF);
        P.own0 = live ? (uint32_t) (d.x - d.w + my_row) * ROWB + my_piece : OOR;
        P.nbl0 = live ? (uint32_t) d.x * (VMHIP_NBL_STRIDE * 2) + (uint32_t) (wave * 64 + lane) * 4 : OOR;
#pragma unroll
        for (int r = 0; r < NRP - NRP_OWN; ++r) {
            const int hi = r * RPR + my_row; /* which halo row */
            const uint32_t hrow = slot[4 + hi];
            P.halo_off[r] = (live && hi < d.z) ? (hrow - (uint32_t) d.w) * ROWB + my_piece : OOR;
        }
    };
    auto fill_item = [&](int i, const Plan& P) {
        if (i < NR) {
            const int plane = i / NRP, r = i % NRP;
            const uint32_t row_off = r < NRP_OWN ? (P.own0 == OOR ? OOR : P.own0 + (uint32_t) (r * RPR * ROWB)) : P.halo_off[r - NRP_OWN];
            load_to_lds_b128(P.in_rsrc, P.base + (uint32_t) (plane * PLANE + (r * 256 + wave * 64) * 16), row_off == OOR ? OOR : row_off + (uint32_t) (plane * 128));
        }
        else if (i < N_FILL) {
            /* the half tile's rows of the neighbour table: 2 KB, 4 bytes per lane and load */
            const uint32_t word = (uint32_t) ((i - NR) * 256);
            load_to_lds_b32(nbl_rsrc, P.base + NBL_AT + (word + wave * 64) * 4, P.nbl0 == OOR ? OOR : P.nbl0 + word * 4);
        }
    };
    auto tile_of = [&](int k) { return tile0 + k * gx; };

    /* ---- prologue: half tile 0 on its way into buffer 0, the note of half tile 1 requested ---- */
    request_note(tile_of(0), true);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    int4 d_next = read_note();
    {
        Plan P;
        plan_fill(d_next, true, 0, P);
#pragma unroll
        for (int i = 0; i < N_FILL; ++i) fill_item(i, P);
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); /* the slot has been read: it may be written again */
    request_note(tile_of(1), 1 < count);

    v16f acc_done[2]; /* the accumulators of the half tile before, waiting for activation and store */
    Done done;
    done.first = 0;
#pragma unroll
    for (int rb = 0; rb < 2; ++rb) {
        done.own[rb] = 0, done.valid[rb] = false;
#pragma unroll
        for (int v = 0; v < 16; ++v) acc_done[rb][v] = 0.0f;
    }

    /* Activation and stores of a finished half tile (lane holds channels cb*32 + h*16 + g*4 + {0..3} of its rows), cut
     * into N_SLICES pieces of a few vector instructions each, so that one piece can follow each matrix instruction of
     * the half tile after: pieces 0..31 apply the activation to one value each, pieces 32..47 convert and store -
     * pieces 32 + 2u and 33 + 2u belong to unit u = (row block, g), and slice_stores says which of them store. The
     * softmax needs the sums of whole rows first, which lie in two waves: prepare_softmax does that part in one go. */
    constexpr int N_SLICES = 48;
    auto prepare_softmax = [&](v16f (&a)[2]) {
#pragma unroll
        for (int rb = 0; rb < 2; ++rb) {
            float sum = 0.0f;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                a[rb][v] = expf(a[rb][v]);
                sum += a[rb][v];
            }
            sum += __shfl_xor(sum, 32);
            if (h == 0) xch[(rh * 64 + rb * 32 + r32) * 2 + cb] = sum;
        }
        __syncthreads();
#pragma unroll
        for (int rb = 0; rb < 2; ++rb) {
            const float2 s2 = *reinterpret_cast<const float2*>(xch + (rh * 64 + rb * 32 + r32) * 2);
            const float inv = 1.0f / (s2.x + s2.y);
#pragma unroll
            for (int v = 0; v < 16; ++v) a[rb][v] = a[rb][v] * inv;
        }
    };
    auto finish_slice = [&](int i, v16f (&a)[2], const Done& t, const __amdgpu_buffer_rsrc_t& rs) {
        if (i < 32) {
            if constexpr (ACT != VMHIP_SOFTMAX) {
                const int rb = i >> 4, v = i & 15;
                const float x = a[rb][v];
                a[rb][v] = ACT == VMHIP_SELU ? selu(x) : ACT == VMHIP_RELU ? fmaxf(x, 0.0f) : fast_tanh(x);
            }
        }
        else if (i < N_SLICES) {
            const int u = (i - 32) >> 1, part = (i - 32) & 1;
            const int rb = u >> 2, g = u & 3;
            /* What one store instruction writes of a row should be as long a run as two lanes can make it: 32 bytes. fp32
             * rows out: matrix column 8 g + 4 h + v is channel 8 g + 4 h + v, a lane's four values of unit g are 16 bytes
             * and the row's other lane holds the next 16. bf16 and hi + lo rows out: the host gives matrix column
             * 8 g + 4 h + v the weights of channel 16 (g / 2) + 8 h + 4 (g % 2) + v, so that a lane's eight values of
             * units g and g + 1 are eight consecutive channels, 16 bytes, and again the other lane holds the next 16
             * (with the columns left as they are a lane had 8 bytes per instruction, the pair 16, and twice the
             * instructions). */
            const int o = cb * 32 + (OUT_FMT == VM_ROWS_F32 ? g * 8 + h * 4 : (g >> 1) * 16 + h * 8);
            if constexpr (OUT_FMT == VM_ROWS_F32) {
                if (part == 0) {
                    const float v0 = a[rb][g * 4 + 0], v1 = a[rb][g * 4 + 1], v2 = a[rb][g * 4 + 2], v3 = a[rb][g * 4 + 3];
                    __builtin_amdgcn_raw_buffer_store_b128(v4u{__float_as_uint(v0), __float_as_uint(v1), __float_as_uint(v2), __float_as_uint(v3)}, rs,
                                                           t.valid[rb] ? t.own[rb] * OUTB + o * 4 : OOR, 0, 0);
                }
            }
            else if (g % 2 == 0) { /* eight channels: units g and g + 1 */
                float v[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) v[e] = a[rb][g * 4 + e];
                const uint32_t h0 = pack_bf16(v[0], v[1]), h1 = pack_bf16(v[2], v[3]), h2 = pack_bf16(v[4], v[5]), h3 = pack_bf16(v[6], v[7]);
                const uint32_t at = t.valid[rb] ? t.own[rb] * OUTB + o * 2 : OOR;
                if (part == 0) {
                    __builtin_amdgcn_raw_buffer_store_b128(v4u{h0, h1, h2, h3}, rs, at, 0, 0);
                }
                else if constexpr (OUT_FMT == VM_ROWS_BF16X2) {
                    const uint32_t l0 = pack_bf16(v[0] - bf16_low(h0), v[1] - bf16_high(h0)), l1 = pack_bf16(v[2] - bf16_low(h1), v[3] - bf16_high(h1));
                    const uint32_t l2 = pack_bf16(v[4] - bf16_low(h2), v[5] - bf16_high(h2)), l3 = pack_bf16(v[6] - bf16_low(h3), v[7] - bf16_high(h3));
                    __builtin_amdgcn_raw_buffer_store_b128(v4u{l0, l1, l2, l3}, rs, t.valid[rb] ? at + CH * 2 : OOR, 0, 0);
                }
            }
        }
    };
    auto out_window = [&](const Done& t) {
        return __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<char*>(out) + (size_t) t.first * OUTB, 0, BT * OUTB, 0x00020000);
    };

    for (int k = 0; k < count; ++k) {
        const int b = k & 1;
        const char* const rows = lds + b * BUF;
        /* my loads of half tile k and the note of k+1 have landed once nothing but the stores issued after them can
         * be in flight (vector memory operations complete in order); before the first stores: once nothing is */
        if (k == 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        else asm volatile("s_waitcnt vmcnt(%0)" ::"n"(stores_after_fills(N_FILL, 48, OUT_FMT)) : "memory");
        __syncthreads(); /* everyone's have landed; everyone has read the last of half tile k-1 */
        const int4 d_cur = d_next;
        d_next = read_note();
        Plan plan; /* the loads of half tile k+1 into the other buffer: issued between the matrix instructions below */
        plan_fill(d_next, k + 1 < count, b ^ 1, plan);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); /* the slot has been read: it may be written again */
        request_note(tile_of(k + 2), k + 2 < count);

        /* the lane's rows and where their gather slots lie in the buffer */
        Done cur;
        cur.first = (uint32_t) d_cur.x;
        uint32_t at[2][SLOTS], xs[2][SLOTS];
        bool far = false;
#pragma unroll
        for (int rb = 0; rb < 2; ++rb) {
            const int own = rh * 64 + rb * 32 + r32;
            cur.valid[rb] = own < d_cur.y;
            cur.own[rb] = (uint32_t) max(0, min(own, d_cur.y - 1)); /* lanes past the rows in use redo the last one and store nothing */
            const v4u nbl = *reinterpret_cast<const v4u*>(rows + NBL_AT + cur.own[rb] * 16);
#pragma unroll
            for (int s = 0; s < SLOTS; ++s) {
                uint32_t li = s == 0 ? cur.own[rb] : nbl_entry(nbl, s - 1);
                far |= li >= (uint32_t) BROWS;
                li = li >= (uint32_t) BROWS ? 0u : li;
                /* a lane's pieces of a half row are (4h + j) ^ swizzle, j = 0..3 (fp32 rows: pieces 2j and 2j + 1 of plane
                 * h): at = the half row, xs = the part of the piece's place that does not depend on j */
                const uint32_t sw = (li >> 1) & 7u;
                at[rb][s] = li * 128u + (IN_FMT == VM_ROWS_F32 ? (uint32_t) (h * PLANE) : 0u);
                xs[rb][s] = IN_FMT == VM_ROWS_F32 ? sw * 16u : ((uint32_t) (h * 4) ^ sw) * 16u;
            }
        }
        const bool any_far = __any(far);

        v16f acc[2];
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const v4f b4 = *reinterpret_cast<const v4f*>(b_lds + cb * 32 + (OUT_FMT == VM_ROWS_F32 ? g * 8 + h * 4 : (g >> 1) * 16 + h * 8 + (g & 1) * 4));
#pragma unroll
            for (int rb = 0; rb < 2; ++rb) acc[rb][g * 4 + 0] = b4[0], acc[rb][g * 4 + 1] = b4[1], acc[rb][g * 4 + 2] = b4[2], acc[rb][g * 4 + 3] = b4[3];
        }

        /* The matrix work, compiled twice: the usual half tile touches nothing but LDS; one with neighbours that are not
         * staged (wave-uniform choice) fetches those lanes' operands from global memory. The activation and stores of
         * the half tile before are part of the same stretch of code so that they are scheduled between the matrix
         * instructions. */
        auto contract = [&](auto far_tag) {
            constexpr bool FAR = decltype(far_tag)::value;
            /* the operands of row block rb for chunk c = (slot, step) */
            auto gather = [&](int c, int rb, v4u& xh, v4u& xl) {
                const int s = c >> 2, j = c & 3;
                const char* const p = rows + at[rb][s];
                if constexpr (IN_FMT == VM_ROWS_BF16) {
                    xh = *reinterpret_cast<const v4u*>(p + (xs[rb][s] ^ (uint32_t) (j * 16)));
                    xl = xh;
                }
                else if constexpr (IN_FMT == VM_ROWS_BF16X2) {
                    /* the lo plane follows the hi plane */
                    const char* const q = p + (xs[rb][s] ^ (uint32_t) (j * 16));
                    xh = *reinterpret_cast<const v4u*>(q);
                    xl = *reinterpret_cast<const v4u*>(q + PLANE);
                }
                else {
                    const v4u f0 = *reinterpret_cast<const v4u*>(p + (xs[rb][s] ^ (uint32_t) (j * 32)));
                    const v4u f1 = *reinterpret_cast<const v4u*>(p + (xs[rb][s] ^ (uint32_t) (j * 32 + 16)));
                    split_eight(f0, f1, xh, xl);
                }
                if constexpr (FAR) {
                    if (s > 0) {
                        const v4u nbl = *reinterpret_cast<const v4u*>(rows + NBL_AT + cur.own[rb] * 16);
                        if (nbl_entry(nbl, s - 1) >= (uint32_t) BROWS) {
                            const int g = B.row_nb[(size_t) (cur.first + cur.own[rb]) * B.nb_stride + (s - 1)];
                            const char* const gp = reinterpret_cast<const char*>(in) + (size_t) ((uint32_t) d_cur.w + (uint32_t) g) * ROWB;
                            if constexpr (IN_FMT == VM_ROWS_BF16) {
                                xh = *reinterpret_cast<const v4u*>(gp + (h * 4 + j) * 16);
                                xl = xh;
                            }
                            else if constexpr (IN_FMT == VM_ROWS_BF16X2) {
                                xh = *reinterpret_cast<const v4u*>(gp + (h * 4 + j) * 16);
                                xl = *reinterpret_cast<const v4u*>(gp + 128 + (h * 4 + j) * 16);
                            }
                            else {
                                const v4u f0 = *reinterpret_cast<const v4u*>(gp + (h * 4 + j) * 32);
                                const v4u f1 = *reinterpret_cast<const v4u*>(gp + (h * 4 + j) * 32 + 16);
                                split_eight(f0, f1, xh, xl);
                            }
                        }
                    }
                }
            };
            if constexpr (ACT == VMHIP_SOFTMAX) prepare_softmax(acc_done);
            const __amdgpu_buffer_rsrc_t rs = out_window(done);
            constexpr int CHUNKS = SLOTS * 4;
            constexpr int PER = WIDE ? 6 : 4;       /* matrix instructions per chunk */
            constexpr int ITEMS = WIDE ? 4 : 3;     /* ... of which so many are followed by an item of the side work */
            static_assert(CHUNKS * ITEMS >= FILL_EVERY * N_FILL + N_SLICES, "every item of the side work finds its place");
            /* The operands of a chunk are requested AHEAD chunks ahead: the four waves ask in step, and an LDS that serves
             * sixteen requests at once (more where lanes collide in a bank) and the loads landing in the other buffer takes
             * some hundred cycles to answer - more than the 128 cycles that a chunk of four matrix instructions lasts. */
            constexpr int AHEAD = WIDE ? 3 : 4, NB = AHEAD + 1;
            v4u xh[NB][2], xl[NB][2];
#pragma unroll
            for (int c = 0; c < AHEAD; ++c) {
                gather(c, 0, xh[c][0], xl[c][0]);
                gather(c, 1, xh[c][1], xl[c][1]);
            }
            static_for<CHUNKS>([&](auto chunk) {
                constexpr int c = decltype(chunk)::value;
                constexpr int s = c >> 2, j = c & 3, u = c % NB, u2 = (c + AHEAD) % NB;
                const v8bf a_hi = __builtin_bit_cast(v8bf, w[s][j][0]), a_lo = __builtin_bit_cast(v8bf, w[s][j][1]);
                /* A wave issues in order and a matrix instruction keeps the pipe busy for 32 cycles: whatever else is
                 * to be done goes between the matrix instructions, a little after each (the scheduling barriers keep
                 * it there). After the first two: the operands of the chunk after, one row block each. After some:
                 * an item of the side work - first the loads of half tile k+1, then the activation and stores of
                 * half tile k-1. */
                static_for<PER>([&](auto mm) {
                    constexpr int m = decltype(mm)::value;
                    constexpr int rb = m & 1;
                    constexpr int kind = m >> 1; /* x_hi * w_hi, then (hi + lo rows) x_lo * w_hi, then x_hi * w_lo */
                    const v8bf a_op = kind == PER / 2 - 1 ? a_lo : a_hi;
                    const v8bf b_op = __builtin_bit_cast(v8bf, (WIDE && kind == 1) ? xl[u][rb] : xh[u][rb]);
                    acc[rb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a_op, b_op, acc[rb], 0, 0, 0);
                    __builtin_amdgcn_sched_barrier(0);
                    if constexpr (m < 2 && c + AHEAD < CHUNKS) gather(c + AHEAD, m, xh[u2][m], xl[u2][m]);
                    if constexpr (m >= PER - ITEMS) {
                        /* every third item is a load until there are no more: issued in a row they fill the memory
                         * pipeline, and the wave stands at the issue of the next */
                        constexpr int item = c * ITEMS + (m - (PER - ITEMS));
                        if constexpr (item % FILL_EVERY == 0 && item / FILL_EVERY < N_FILL) fill_item(item / FILL_EVERY, plan);
                        else if constexpr (slice_of_item(item, N_FILL) < N_SLICES) finish_slice(slice_of_item(item, N_FILL), acc_done, done, rs);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                });
            });
        };
        if (any_far) {
            contract(std::true_type());
            /* the side path's loads are not part of the count above: none may be in flight when the next wait counts */
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        }
        else {
            contract(std::false_type());
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); /* every operand of the half tile has been read */
#pragma unroll
        for (int rb = 0; rb < 2; ++rb) acc_done[rb] = acc[rb];
        done = cur;
    }
    /* the last half tile's results; and no LDS load may outlive the wave */
    __syncthreads(); /* the exchange area of the softmax is free again */
    if constexpr (ACT == VMHIP_SOFTMAX) prepare_softmax(acc_done);
    {
        const __amdgpu_buffer_rsrc_t rs = out_window(done);
#pragma unroll
        for (int i = 0; i < N_SLICES; ++i) finish_slice(i, acc_done, done, rs);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

/* ---- half-tile tables ---- */

/* active_h[f] = half tiles in use of the frames before f (a frame uses ceil((V + 1) / 128): its visible rows and the
 * null row); one block */
__global__ __launch_bounds__(256) void vm_half_prefix_kernel(VmBatchDev B) {
    __shared__ int wave_total[4];
    __shared__ int carry_s;
    if (threadIdx.x == 0) carry_s = 0;
    __syncthreads();
    for (int base = 0; base < B.n_frames; base += 256) {
        const int f = base + (int) threadIdx.x;
        const int mine = f < B.n_frames ? (B.frame_V[f] + 1 + BT - 1) / BT : 0;
        int scan = mine;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const int up = __shfl_up(scan, d);
            if ((int) (threadIdx.x & 63) >= d) scan += up;
        }
        if ((threadIdx.x & 63) == 63) wave_total[threadIdx.x >> 6] = scan;
        __syncthreads();
        int before = carry_s + scan - mine;
        for (int wv = 0; wv < (int) (threadIdx.x >> 6); ++wv) before += wave_total[wv];
        if (f < B.n_frames) B.active_h[f] = before;
        __syncthreads();
        if (threadIdx.x == 255) carry_s = before + mine;
        __syncthreads();
    }
    if (threadIdx.x == 0) B.active_h[B.n_frames] = carry_s;
}

/* One block per half tile of the row space: the neighbours (B.row_nb, frame-local rows) that live in other half tiles
 * are deduplicated through an open-addressing hash in LDS and numbered densely in table order (the halo slots), every
 * neighbour is rewritten as a position in "own half tile's rows, then halo slots", and the half tile's note is
 * written at its number among the half tiles in use. Which row gets which halo slot depends on the order the atomics
 * land in and may differ from run to run; the rows a slot stands for, and so every result, do not. */
#define HB_HASH 2048 /* >= the most out-of-tile neighbours a half tile can have (128 rows x 8) */
__global__ __launch_bounds__(BT) void vm_half_tables_kernel(VmBatchDev B) {
    __shared__ __align__(16) uint32_t h_key[HB_HASH];
    __shared__ uint16_t h_dense[HB_HASH];
    __shared__ int wave_total[BT / 64];
    __shared__ __align__(16) uint16_t nbl_rows[BT][VMHIP_NBL_STRIDE];

    const int tile = blockIdx.x >> 1;
    if (tile >= vm_row_tiles(B)) return; /* the grid may be sized for more tiles than the staged batch has */
    const int f = find_frame_by_row_tile(B.frames, B.n_frames, tile);
    const VmFrame& F = B.frames[f];
    const int V = B.frame_V[f];
    const int nn = F.nn;
    const int row0 = (tile - F.row_tile0) * VMHIP_TILE + (int) (blockIdx.x & 1) * BT;
    const int n_rows = max(0, min(BT, V + 1 - row0));
    if (n_rows == 0) return;
    const int number = B.active_h[f] + row0 / BT;
    uint32_t* const note = B.tile_note_h + (size_t) number * NOTE;

    constexpr uint32_t EMPTY = 0xffffffffu;
    auto hash = [](uint32_t key) { return (key * 2654435761u) >> 21; }; /* 11 bits */
    for (int e = threadIdx.x * 4; e < HB_HASH; e += BT * 4) *reinterpret_cast<uint4*>(&h_key[e]) = make_uint4(EMPTY, EMPTY, EMPTY, EMPTY);
    __syncthreads();

    /* thread = row; its neighbours stay in registers between the passes */
    const bool mine = (int) threadIdx.x < n_rows;
    int nb[VMHIP_NBL_STRIDE];
#pragma unroll
    for (int j = 0; j < VMHIP_NBL_STRIDE; ++j) {
        nb[j] = (mine && j < nn) ? B.row_nb[((size_t) F.row_base + row0 + threadIdx.x) * B.nb_stride + j] : -1;
        if (nb[j] >= 0 && (nb[j] < row0 || nb[j] >= row0 + BT)) {
            uint32_t slot = hash((uint32_t) nb[j]);
            while (true) {
                const uint32_t prev = atomicCAS(&h_key[slot], EMPTY, (uint32_t) nb[j]);
                if (prev == EMPTY || prev == (uint32_t) nb[j]) break;
                slot = (slot + 1) & (HB_HASH - 1);
            }
        }
    }
    __syncthreads();

    /* dense numbering of the occupied hash entries, in table order: 16 entries per thread, block-wide scan */
    constexpr int PER = HB_HASH / BT;
    uint32_t keys[PER];
#pragma unroll
    for (int k = 0; k < PER; k += 4) {
        const uint4 t = *reinterpret_cast<const uint4*>(&h_key[threadIdx.x * PER + k]);
        keys[k] = t.x, keys[k + 1] = t.y, keys[k + 2] = t.z, keys[k + 3] = t.w;
    }
    int have = 0;
#pragma unroll
    for (int k = 0; k < PER; ++k) have += keys[k] != EMPTY;
    int scan = have;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const int up = __shfl_up(scan, d);
        if ((int) (threadIdx.x & 63) >= d) scan += up;
    }
    if ((threadIdx.x & 63) == 63) wave_total[threadIdx.x >> 6] = scan;
    __syncthreads();
    int before = scan - have, total = 0;
#pragma unroll
    for (int wv = 0; wv < BT / 64; ++wv) {
        if (wv < (int) (threadIdx.x >> 6)) before += wave_total[wv];
        total += wave_total[wv];
    }
    const int cap = min(B.halo_cap, BH);
    if (have > 0) {
#pragma unroll
        for (int k = 0; k < PER; ++k) {
            if (keys[k] != EMPTY) {
                h_dense[threadIdx.x * PER + k] = (uint16_t) min(before, 0xffff);
                if (before < cap) note[4 + before] = (uint32_t) F.row_base + keys[k];
                ++before;
            }
        }
    }
    if (threadIdx.x == 0) {
        note[0] = (uint32_t) (F.row_base + row0), note[1] = (uint32_t) n_rows, note[2] = (uint32_t) min(total, cap), note[3] = (uint32_t) F.row_base;
    }
    __syncthreads();

    if (mine) {
#pragma unroll
        for (int j = 0; j < VMHIP_NBL_STRIDE; ++j) {
            uint32_t local = 0;
            if (nb[j] >= 0) {
                if (nb[j] >= row0 && nb[j] < row0 + BT) {
                    local = (uint32_t) (nb[j] - row0);
                }
                else {
                    uint32_t slot = hash((uint32_t) nb[j]);
                    while (h_key[slot] != (uint32_t) nb[j]) slot = (slot + 1) & (HB_HASH - 1);
                    const int dense = h_dense[slot];
                    local = dense < cap ? (uint32_t) (BT + dense) : VMHIP_NBL_FAR;
                }
            }
            nbl_rows[threadIdx.x][j] = (uint16_t) local;
        }
        *reinterpret_cast<uint4*>(B.row_nbl_h + ((size_t) F.row_base + row0 + threadIdx.x) * VMHIP_NBL_STRIDE) = *reinterpret_cast<const uint4*>(nbl_rows[threadIdx.x]);
    }
}

template <int SLOTS, int IN_FMT, int OUT_FMT, int ACT>
int launch_bf16(const VmBatchDev& B, const VmLayerDev& L, const void* in, void* out, hipStream_t stream) {
    constexpr size_t lds = bf16_lds_bytes(IN_FMT);
    static_assert(lds <= 160 * 1024, "two row buffers must fit the CU's LDS");
    auto kernel = vm_conv_bf16_kernel<SLOTS, IN_FMT, OUT_FMT, ACT>;
    static std::atomic<bool> configured{false}; /* engines on several host threads may get here together */
    if (!configured) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, int(lds)) != hipSuccess) {
            (void) hipGetLastError();
            return -1;
        }
        configured = true;
    }
    /* one block of four waves per CU; the kernel reads the number of half tiles in use on the device */
    hipLaunchKernelGGL(kernel, dim3(256), dim3(256), lds, stream, B, L, in, out);
    return 0;
}

uint16_t bf16_round(float f) {
    uint32_t u;
    std::memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return uint16_t((u >> 16) | 0x40); /* NaN stays NaN */
    u += 0x7fffu + ((u >> 16) & 1u);                                         /* round to nearest even */
    return uint16_t(u >> 16);
}

}  // namespace

/* Weight layout the kernel consumes: [channel block cb][slot][step j][part: hi, lo][lane = h*32 + o][e = 0..7] bf16 of
 * W[slot*64 + (4h + j)*8 + e][cb*32 + channel(o)]. The matrix instruction leaves a lane columns 8 g + 4 h' + v (g = 0..3,
 * v = 0..3) of its row; for a layer that writes fp32 rows channel(o) = o, for one that writes bf16 or hi + lo rows
 * channel(8 g + 4 h' + v) = 16 (g / 2) + 8 h' + 4 (g % 2) + v (the kernel's store says why). */
size_t vm_bf16_weight_bytes(int c_in, int c_out, int slots) { return size_t(slots) * (c_in / 16) * (c_out / 32) * 2 * 64 * 16; }
void vm_bf16_permute_weights(const float* w, int c_in, int c_out, int slots, int out_fmt, void* wp) {
    uint16_t* dst = reinterpret_cast<uint16_t*>(wp);
    const int steps = c_in / 16, cbs = c_out / 32;
    for (int cb = 0; cb < cbs; ++cb)
        for (int s = 0; s < slots; ++s)
            for (int j = 0; j < steps; ++j)
                for (int h = 0; h < 2; ++h)
                    for (int o = 0; o < 32; ++o)
                        for (int e = 0; e < 8; ++e) {
                            const int k = s * c_in + (h * steps + j) * 8 + e;
                            const int g = o >> 3, hh = (o >> 2) & 1, vv = o & 3;
                            const int channel = out_fmt == VM_ROWS_F32 ? o : (g >> 1) * 16 + hh * 8 + (g & 1) * 4 + vv;
                            const float v = w[size_t(k) * c_out + cb * 32 + channel];
                            const uint16_t hi = bf16_round(v);
                            const uint32_t hi_bits = uint32_t(hi) << 16;
                            float hi_f;
                            std::memcpy(&hi_f, &hi_bits, 4);
                            const uint16_t lo = std::isfinite(v) ? bf16_round(v - hi_f) : uint16_t(0);
                            const size_t at = ((size_t(cb) * slots + s) * steps + j) * 2;
                            dst[((at + 0) * 64 + h * 32 + o) * 8 + e] = hi;
                            dst[((at + 1) * 64 + h * 32 + o) * 8 + e] = lo;
                        }
}

bool vm_bf16_supported(int c_in, int c_out, int slots) { return c_in == CH && c_out == CH && slots == 7; }

void vm_launch_half_tables(const VmBatchDev& B, hipStream_t stream) {
    if (B.n_row_tiles <= 0 || !B.row_nbl_h) return;
    hipLaunchKernelGGL(vm_half_prefix_kernel, dim3(1), dim3(256), 0, stream, B);
    hipLaunchKernelGGL(vm_half_tables_kernel, dim3(2 * B.n_row_tiles), dim3(BT), 0, stream, B);
}

int vm_launch_conv_bf16(const VmBatchDev& B, const VmLayerDev& L, const void* in, void* out, hipStream_t stream, const char** kernel_name) {
    if (B.n_row_tiles <= 0) return 0;
    if (!B.row_nbl_h || !B.tile_note_h || !B.active_h || !L.w_mfma || !vm_bf16_supported(L.c_in, L.c_out, L.slots)) return -1;
    /* the kernel addresses a frame's input rows with 32-bit byte offsets: a batch with a frame of 2^24 rows or more is
     * refused when it is staged for an engine with such layers (api.hip) */
#define Z(FI, FO, ACT, NAME)                                                       \
    if (L.in_bf16 == FI && L.out_bf16 == FO && L.activation == ACT) {              \
        if (kernel_name) *kernel_name = NAME;                                      \
        return launch_bf16<7, FI, FO, ACT>(B, L, in, out, stream);                 \
    }
#define Y(FI, FO, NAME)                  \
    Z(FI, FO, VMHIP_SELU, NAME)          \
    Z(FI, FO, VMHIP_RELU, NAME)          \
    Z(FI, FO, VMHIP_TANH, NAME)          \
    Z(FI, FO, VMHIP_SOFTMAX, NAME)
    Y(VM_ROWS_BF16X2, VM_ROWS_BF16X2, "conv_bf16_x2_tox2_64x64s7")
    Y(VM_ROWS_BF16X2, VM_ROWS_BF16, "conv_bf16_x2_tobf16_64x64s7")
    Y(VM_ROWS_BF16X2, VM_ROWS_F32, "conv_bf16_x2_tof32_64x64s7")
    Y(VM_ROWS_BF16, VM_ROWS_BF16X2, "conv_bf16_bf16_tox2_64x64s7")
    Y(VM_ROWS_BF16, VM_ROWS_BF16, "conv_bf16_bf16_tobf16_64x64s7")
    Y(VM_ROWS_BF16, VM_ROWS_F32, "conv_bf16_bf16_tof32_64x64s7")
    Y(VM_ROWS_F32, VM_ROWS_BF16X2, "conv_bf16_f32_tox2_64x64s7")
    Y(VM_ROWS_F32, VM_ROWS_BF16, "conv_bf16_f32_tobf16_64x64s7")
    Y(VM_ROWS_F32, VM_ROWS_F32, "conv_bf16_f32_tof32_64x64s7")
#undef Y
#undef Z
    return -1;
}
